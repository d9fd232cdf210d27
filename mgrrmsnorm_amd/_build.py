"""Build recipe for libmegagemm_hip.so (hipcc, gfx950 only).

The library is built in-tree, next to this file, so that a built copy travels with the
source tree.  `python -m mgrrmsnorm_amd._build` rebuilds it; `build()` is what the
package's own entry points call.  Replaces the reference's CUDAExtension recipe
(setup.py:23-41) and its Makefile (Makefile:9-26).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libmegagemm_hip.so"
OBJ_DIR = PKG_DIR / "csrc" / "_obj"

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


def build(jobs: int | None = None, verbose: bool = False) -> Path:
    """Compile every translation unit for gfx950 and link libmegagemm_hip.so."""
    hipcc = find_hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs = []

    def compile_one(unit):
        src, stem, defs = unit
        obj = OBJ_DIR / f"{stem}.o"
        cmd = [hipcc, *COMMON_FLAGS, *defs, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, UNITS))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv)
    print(f"built {path}")
