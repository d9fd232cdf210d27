"""Compile tests/integration/torch_binding.cpp into an importable torch extension module
(`mg_torch_binding`) next to this file: host-only C++ (g++), linked against torch and the
prebuilt libmegagemm_hip.so.  Usage: python tests/integration/build_binding.py"""
from __future__ import annotations

import subprocess
import sys
import sysconfig
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
NAME = "mg_torch_binding"
TARGET = HERE / f"{NAME}{sysconfig.get_config_var('EXT_SUFFIX')}"


def build() -> Path:
    import torch
    from torch.utils import cpp_extension as ce

    lib_dir = ROOT / "mgrrmsnorm_amd"
    if not (lib_dir / "libmegagemm_hip.so").exists():
        raise RuntimeError("build libmegagemm_hip.so first: python -m mgrrmsnorm_amd._build")
    torch_libs = ce.library_paths()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{ROOT / 'include'}", *[f"-I{p}" for p in ce.include_paths()],
           f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include",
           str(HERE / "torch_binding.cpp"), "-o", str(TARGET),
           *[f"-L{p}" for p in torch_libs], "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip",
           "-ltorch_hip", f"-L{lib_dir}", "-lmegagemm_hip", "-Wl,-rpath,$ORIGIN/../../mgrrmsnorm_amd",
           *[f"-Wl,-rpath,{p}" for p in torch_libs]]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed:\n" + proc.stdout)
    return TARGET


if __name__ == "__main__":
    print(f"built {build()}")
    sys.exit(0)
