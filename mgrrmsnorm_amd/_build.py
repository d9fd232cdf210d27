"""Build recipe for libmegagemm_hip.so (hipcc, gfx950 only) and for the torch extension
over it (`_binding`, host-only C++ compiled with g++).

Both are built in-tree, next to this file, so that built copies travel with the source
tree.  `python -m mgrrmsnorm_amd._build` rebuilds them; `build()` is what the package's own
entry points call.  Replaces the reference's CUDAExtension recipe (setup.py:23-41) and its
Makefile (Makefile:9-26).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libmegagemm_hip.so"
OBJ_DIR = PKG_DIR / "csrc" / "_obj"

BINDING_NAME = "_binding"
BINDING_PATH = PKG_DIR / f"{BINDING_NAME}{sysconfig.get_config_var('EXT_SUFFIX')}"

ARCH = "gfx950"

# (source, object stem, extra defines)
UNITS = [
    ("mg_api.hip", "mg_api", []),
    ("swiglu_inst.hip", "swiglu_inst", []),
    ("rmsnorm_fwd_inst.hip", "rmsnorm_fwd_f32", ["-DMG_DTYPE=0"]),
    ("rmsnorm_fwd_inst.hip", "rmsnorm_fwd_f16", ["-DMG_DTYPE=1"]),
    ("rmsnorm_fwd_inst.hip", "rmsnorm_fwd_bf16", ["-DMG_DTYPE=2"]),
    ("rmsnorm_bwd_inst.hip", "rmsnorm_bwd_f32", ["-DMG_DTYPE=0"]),
    ("rmsnorm_bwd_inst.hip", "rmsnorm_bwd_f16", ["-DMG_DTYPE=1"]),
    ("rmsnorm_bwd_inst.hip", "rmsnorm_bwd_bf16", ["-DMG_DTYPE=2"]),
]

# Packed fp32 VALU instructions are switched off for all device code.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-Wall",
                f"-I{INCLUDE}", f"-I{CSRC}"] + DEVICE_FLAGS


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), proc.stdout))
    # hipcc's host pass does not know the device-only target feature and says so; drop that line
    noise = "is not a recognized feature for this target"
    rest = [ln for ln in proc.stdout.splitlines() if ln.strip() and noise not in ln]
    if rest:
        sys.stderr.write("\n".join(rest) + "\n")


def build_binding(verbose: bool = False, out_dir: Path | None = None, lib_dir: Path | None = None) -> Path:
    """Compile csrc/torch_binding.cpp into the extension module `_binding`: plain C++ built
    with g++ against torch's headers and libraries and linked to libmegagemm_hip.so, which it
    finds next to itself at run time ($ORIGIN)."""
    import torch
    from torch.utils import cpp_extension as ce

    lib_dir = lib_dir or PKG_DIR
    target = (out_dir or PKG_DIR) / BINDING_PATH.name
    if not (lib_dir / LIB_PATH.name).exists():
        raise RuntimeError(f"build {LIB_PATH.name} first")
    cxx = os.environ.get("CXX") or shutil.which("g++")
    if not cxx:
        raise RuntimeError("no C++ compiler found (looked at $CXX and g++)")
    torch_libs = ce.library_paths()
    tmp = target.with_suffix(".so.tmp")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={BINDING_NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{INCLUDE}", *[f"-I{p}" for p in ce.include_paths()],
           f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include",
           str(CSRC / "torch_binding.cpp"), "-o", str(tmp),
           *[f"-L{p}" for p in torch_libs], "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip",
           "-ltorch_hip", f"-L{lib_dir}", "-lmegagemm_hip", "-Wl,-rpath,$ORIGIN",
           *[f"-Wl,-rpath,{p}" for p in torch_libs]]
    if verbose:
        print(" ".join(cmd), flush=True)
    _run(cmd)
    os.replace(tmp, target)
    return target


def build(jobs: int | None = None, verbose: bool = False, binding: bool = True, out_dir: Path | None = None) -> Path:
    """Compile every translation unit for gfx950, link libmegagemm_hip.so, then build the
    torch extension over it (binding=False skips that: the ctypes binding needs no compiler
    beyond hipcc).  out_dir: where the two files (and the intermediate objects) go instead of
    the package directory."""
    hipcc = find_hipcc()
    out_dir = Path(out_dir) if out_dir else None
    obj_dir = (out_dir / "_obj") if out_dir else OBJ_DIR
    lib_path = (out_dir / LIB_PATH.name) if out_dir else LIB_PATH
    obj_dir.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs = []

    def compile_one(unit):
        src, stem, defs = unit
        obj = obj_dir / f"{stem}.o"
        cmd = [hipcc, *COMMON_FLAGS, *defs, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, UNITS))
    tmp = lib_path.with_suffix(".so.tmp")
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)])
    os.replace(tmp, lib_path)
    if binding:
        build_binding(verbose=verbose, out_dir=out_dir, lib_dir=out_dir)
    return lib_path


def is_current() -> bool:
    """True when both built files exist and are newer than every source they are made from
    (csrc/*.hip, *.hpp, *.cpp, include/*.h and this recipe)."""
    outs = [LIB_PATH, BINDING_PATH]
    if not all(p.exists() for p in outs):
        return False
    srcs = [*CSRC.glob("*.hip"), *CSRC.glob("*.hpp"), *CSRC.glob("*.cpp"), *INCLUDE.glob("*.h"), Path(__file__)]
    return min(p.stat().st_mtime for p in outs) >= max(p.stat().st_mtime for p in srcs)


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv, binding="--no-binding" not in sys.argv)
    print(f"built {path}" + ("" if "--no-binding" in sys.argv else f" and {BINDING_PATH}"))
