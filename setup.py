"""Packaging for mgrrmsnorm_amd: `pip install -e .` (or `python setup.py build`) compiles
libmegagemm_hip.so for gfx950 with hipcc and the torch extension `_binding` over its C ABI
(include/megagemm_hip.h) with g++, and ships both inside the package, next to the ctypes
loader that serves when no C++ compiler is at hand.  `python setup.py build_hip
[--out-dir DIR]` runs just that compile step.  (Reference: a CUDAExtension built by nvcc,
setup.py:23-41.)
"""
import sys
from pathlib import Path

from setuptools import Command, setup
from setuptools.command.build_py import build_py
from setuptools.command.develop import develop

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))


def _compile_library(out_dir=None, only_if_stale=False):
    from mgrrmsnorm_amd import _build

    if only_if_stale and out_dir is None and _build.is_current():
        print(f"{_build.LIB_PATH.name} and {_build.BINDING_PATH.name} are newer than their sources: not rebuilt")
        return
    print(f"building {_build.LIB_PATH.name} for {_build.ARCH} and {_build.BINDING_PATH.name}"
          + (f" into {out_dir}" if out_dir else ""))
    _build.build(out_dir=out_dir)


class BuildHip(Command):
    description = "compile libmegagemm_hip.so with hipcc (gfx950) and the torch extension over it"
    user_options = [("out-dir=", None, "directory for the built files (default: inside the package)")]

    def initialize_options(self):
        self.out_dir = None

    def finalize_options(self):
        pass

    def run(self):
        _compile_library(self.out_dir)


class BuildPyWithHip(build_py):
    """`pip install .` / `python setup.py build`: compile in the source tree (unless what is
    there is newer than its sources), then let build_py copy package data, the built files
    among them."""

    def run(self):
        _compile_library(only_if_stale=True)
        super().run()


class DevelopWithHip(develop):
    """`pip install -e .`: the same compile step; the package then runs from the source tree."""

    def run(self):
        _compile_library(only_if_stale=True)
        super().run()


setup(
    name="mgrrmsnorm-amd",
    version="0.1.0",
    description=("RMSNorm and SwiGLU activation as hand-written HIP kernels for AMD MI355X (gfx950), "
                 "with the Python surface of MadrasLe/MGRrmsnorm's megagemm package"),
    long_description=(ROOT / "README.md").read_text(),
    long_description_content_type="text/markdown",
    license="MIT",
    python_requires=">=3.9",
    install_requires=["torch>=2.0"],
    extras_require={"dev": ["pytest", "numpy"]},
    packages=["mgrrmsnorm_amd", "megagemm"],
    py_modules=["rmsnorm_cuda_ops"],
    package_data={"mgrrmsnorm_amd": ["libmegagemm_hip.so", "_binding*.so", "csrc/*.hip", "csrc/*.hpp", "csrc/*.cpp"]},
    data_files=[("include", ["include/megagemm_hip.h", "include/megagemm_hip_tuning.h"])],
    cmdclass={"build_hip": BuildHip, "build_py": BuildPyWithHip, "develop": DevelopWithHip},
)
