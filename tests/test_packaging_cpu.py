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


@pytest.fixture(scope="module")
def installed(tmp_path_factory):
    """`pip install <copy of the source tree> --target <scratch>`: the whole install path of the
    package -- the build_py hook compiles both files in the (pristine) copy, the wheel carries
    them with the kernel sources, the headers go to <prefix>/include.  (Reference:
    `pip install -e .`, README.md:63-64, setup.py:10-72.)"""
    import shutil

    base = tmp_path_factory.mktemp("mg_install")
    src, site = base / "src", base / "site"
    tracked = subprocess.run(["git", "ls-files"], cwd=ROOT, stdout=subprocess.PIPE, text=True, check=True).stdout.split()
    for rel in tracked:
        if rel.startswith(("mgrrmsnorm_amd/", "megagemm/", "include/")) or rel in (
                "setup.py", "pyproject.toml", "MANIFEST.in", "README.md", "Makefile", "rmsnorm_cuda_ops.py"):
            (src / rel).parent.mkdir(parents=True, exist_ok=True)
            shutil.copy2(ROOT / rel, src / rel)
    assert not list(src.rglob("*.so")), "the copy must start without built files"
    proc = subprocess.run([sys.executable, "-m", "pip", "install", "--no-build-isolation", "--no-deps", "--no-index",
                           "--target", str(site), str(src)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    assert proc.returncode == 0, proc.stdout[-4000:]
    return src, site


def test_pip_install_builds_and_ships_everything(installed):
    from mgrrmsnorm_amd import _build, _lib

    src, site = installed
    pkg = site / "mgrrmsnorm_amd"
    lib_path = pkg / _build.LIB_PATH.name
    assert lib_path.exists() and (pkg / _build.BINDING_PATH.name).exists()
    lib = ctypes.CDLL(str(lib_path))
    lib.mg_abi_version.restype = ctypes.c_int
    assert lib.mg_abi_version() == _lib.ABI_VERSION
    for name in ("mg_api.hip", "rmsnorm_kernels.hpp", "torch_binding.cpp"):
        assert (pkg / "csrc" / name).exists(), f"csrc/{name} did not ship"
    for name in ("megagemm_hip.h", "megagemm_hip_tuning.h"):
        assert (site / "include" / name).exists(), f"include/{name} did not ship"
    assert (site / "megagemm" / "__init__.py").exists() and (site / "rmsnorm_cuda_ops.py").exists()
    # the installed copy imports on its own and finds its library next to itself
    code = ("import sys; sys.path.insert(0, sys.argv[1]); import mgrrmsnorm_amd, megagemm; from mgrrmsnorm_amd import _lib, ops; "
            "assert str(_lib.LIB_PATH).startswith(sys.argv[1]); _lib.load(); print(ops.backend(), megagemm.__version__)")
    proc = subprocess.run([sys.executable, "-c", code, str(site)], cwd=site, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0 and proc.stdout.split()[-2:] == ["extension", "0.1.0"], proc.stdout[-2000:]


def test_develop_hook_runs_and_keeps_a_current_build(installed):
    """`python setup.py develop` (what `pip install -e .` runs) on the copy the previous test
    built: the hook finds both files newer than their sources and does not rebuild; the package
    is then importable from the source tree through the egg-link."""
    src, _ = installed
    target = src.parent / "dev_site"
    target.mkdir()
    before = (src / "mgrrmsnorm_amd" / "libmegagemm_hip.so").stat().st_mtime
    env = dict(**__import__("os").environ, PYTHONPATH=str(target))
    proc = subprocess.run([sys.executable, "setup.py", "develop", "--no-deps", "--install-dir", str(target)], cwd=src,
                          env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "not rebuilt" in proc.stdout
    assert (src / "mgrrmsnorm_amd" / "libmegagemm_hip.so").stat().st_mtime == before
    assert any(p.suffix == ".egg-link" for p in target.iterdir())


def test_package_metadata_lists_what_ships():
    text = (ROOT / "setup.py").read_text()
    for needle in ("libmegagemm_hip.so", "_binding*.so", "megagemm_hip_tuning.h", '"megagemm"', "rmsnorm_cuda_ops"):
        assert needle in text
    assert "csrc/tools" not in text
    manifest = (ROOT / "MANIFEST.in").read_text()
    assert "*.cpp" in manifest and "include/*.h" in manifest
