"""numpy/ctypes front end of the C oracle (mg_oracle.c) plus the rounding helpers that
turn its double-precision answers into the bit patterns an fp32 / fp16 / bf16 kernel
output is compared with.

TEST INFRASTRUCTURE ONLY: see mg_oracle.c for what is restated from where.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "libmg_oracle.so"
_lib = None


def build(force: bool = False) -> Path:
    """Compile mg_oracle.c with gcc (through the Makefile beside it)."""
    src = _DIR / "mg_oracle.c"
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-s", "-B", "-C", str(_DIR), "libmg_oracle.so"], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        p = ctypes.c_void_p
        i64 = ctypes.c_int64
        lib.oracle_rmsnorm_fwd_f32.argtypes = [p, p, p, p, i64, i64, ctypes.c_float]
        lib.oracle_rmsnorm_fwd_f64.argtypes = [p, p, p, p, i64, i64, ctypes.c_double]
        lib.oracle_rmsnorm_bwd_f32.argtypes = [p, p, p, p, p, p, i64, i64]
        lib.oracle_rmsnorm_bwd_f64.argtypes = [p, p, p, p, p, i64, i64, ctypes.c_double]
        for name in ("oracle_swiglu_fwd_f32", "oracle_swiglu_fwd_f64"):
            getattr(lib, name).argtypes = [p, p, i64, i64]
        for name in ("oracle_swiglu_bwd_f32", "oracle_swiglu_bwd_f64"):
            getattr(lib, name).argtypes = [p, p, p, i64, i64]
        _lib = lib
    return _lib


def _f32(a) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _check_2d(x: np.ndarray, name: str):
    if x.ndim != 2:
        raise ValueError(f"{name} must be 2-D, got shape {x.shape}")


# ------------------------------------------------------------------------------ RMSNorm

def rmsnorm_fwd_f32(x, w, eps):
    """Literal fp32 restatement (rmsnorm_standalone.cu:17-30). Returns (y, inv_rms)."""
    x, w = _f32(x), _f32(w)
    _check_2d(x, "x")
    rows, cols = x.shape
    assert w.shape == (cols,)
    y = np.empty_like(x)
    s = np.empty(rows, dtype=np.float32)
    _load().oracle_rmsnorm_fwd_f32(_ptr(y), _ptr(s), _ptr(x), _ptr(w), rows, cols, float(eps))
    return y, s


def rmsnorm_fwd_f64(x, w, eps):
    """Double-precision evaluation from fp32 inputs. Returns (y, inv_rms) as float64."""
    x, w = _f32(x), _f32(w)
    _check_2d(x, "x")
    rows, cols = x.shape
    assert w.shape == (cols,)
    y = np.empty(x.shape, dtype=np.float64)
    s = np.empty(rows, dtype=np.float64)
    _load().oracle_rmsnorm_fwd_f64(_ptr(y), _ptr(s), _ptr(x), _ptr(w), rows, cols, float(eps))
    return y, s


def rmsnorm_bwd_f32(dy, x, w, inv_rms):
    """Literal fp32 restatement (src/rmsnorm_kernel.cu:258-312). Returns (dx, dW)."""
    dy, x, w, inv_rms = _f32(dy), _f32(x), _f32(w), _f32(inv_rms)
    _check_2d(x, "x")
    rows, cols = x.shape
    assert dy.shape == x.shape and w.shape == (cols,) and inv_rms.shape == (rows,)
    dx = np.empty_like(x)
    dw = np.empty(cols, dtype=np.float32)
    _load().oracle_rmsnorm_bwd_f32(_ptr(dx), _ptr(dw), _ptr(dy), _ptr(x), _ptr(w), _ptr(inv_rms), rows, cols)
    return dx, dw


def rmsnorm_bwd_f64(dy, x, w, eps):
    """Double-precision backward from fp32 inputs. Returns (dx, dW) as float64."""
    dy, x, w = _f32(dy), _f32(x), _f32(w)
    _check_2d(x, "x")
    rows, cols = x.shape
    assert dy.shape == x.shape and w.shape == (cols,)
    dx = np.empty(x.shape, dtype=np.float64)
    dw = np.empty(cols, dtype=np.float64)
    _load().oracle_rmsnorm_bwd_f64(_ptr(dx), _ptr(dw), _ptr(dy), _ptr(x), _ptr(w), rows, cols, float(eps))
    return dx, dw


# ------------------------------------------------------------------------------- SwiGLU

def _swiglu_fwd(fn_name, out_dtype, gu):
    gu = _f32(gu)
    _check_2d(gu, "gu")
    M, H2 = gu.shape
    assert H2 % 2 == 0
    H = H2 // 2
    h = np.empty((M, H), dtype=out_dtype)
    getattr(_load(), fn_name)(_ptr(h), _ptr(gu), M, H)
    return h


def _swiglu_bwd(fn_name, out_dtype, dh, gu):
    dh, gu = _f32(dh), _f32(gu)
    _check_2d(gu, "gu")
    M, H2 = gu.shape
    H = H2 // 2
    assert dh.shape == (M, H)
    dgu = np.empty((M, H2), dtype=out_dtype)
    getattr(_load(), fn_name)(_ptr(dgu), _ptr(dh), _ptr(gu), M, H)
    return dgu


def swiglu_fwd_f32(gu):
    return _swiglu_fwd("oracle_swiglu_fwd_f32", np.float32, gu)


def swiglu_fwd_f64(gu):
    return _swiglu_fwd("oracle_swiglu_fwd_f64", np.float64, gu)


def swiglu_bwd_f32(dh, gu):
    return _swiglu_bwd("oracle_swiglu_bwd_f32", np.float32, dh, gu)


def swiglu_bwd_f64(dh, gu):
    return _swiglu_bwd("oracle_swiglu_bwd_f64", np.float64, dh, gu)


# --------------------------------------------------------------- storage-type helpers
# Arrays of fp16 values are numpy float16; arrays of bf16 values are carried as uint16 bit
# patterns (numpy has no bfloat16).

def to_f32(a, dtype: str) -> np.ndarray:
    """Exact widening of stored values to float32. dtype in {'fp32','fp16','bf16'}."""
    if dtype == "fp32":
        return np.asarray(a, dtype=np.float32)
    if dtype == "fp16":
        return np.asarray(a, dtype=np.float16).astype(np.float32)
    if dtype == "bf16":
        bits = np.asarray(a, dtype=np.uint16).astype(np.uint32) << np.uint32(16)
        return bits.view(np.float32)
    raise ValueError(dtype)


def _f64_to_f32_round_to_odd(d: np.ndarray) -> np.ndarray:
    """float64 -> float32 bit patterns rounded to odd (the sticky rounding that makes a
    second round-to-nearest-even, to a narrower type, come out as a single rounding)."""
    d = np.asarray(d, dtype=np.float64)
    with np.errstate(over="ignore"):
        f = d.astype(np.float32)
    bits = f.view(np.uint32).copy()
    back = f.astype(np.float64)
    finite = np.isfinite(d) & np.isfinite(back)
    inexact = finite & (back != d)
    too_big = inexact & (np.abs(back) > np.abs(d))
    bits[too_big] -= np.uint32(1)          # step the magnitude down to the truncated value
    bits[inexact] |= np.uint32(1)          # sticky bit
    return bits


def round_to(d, dtype: str) -> np.ndarray:
    """Round float64 values once, to nearest even, to the storage type.
    Returns float32 for 'fp32', float16 for 'fp16', uint16 bit patterns for 'bf16'."""
    d = np.asarray(d, dtype=np.float64)
    if dtype == "fp32":
        return d.astype(np.float32)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return d.astype(np.float16)
    if dtype == "bf16":
        bits = _f64_to_f32_round_to_odd(d).astype(np.uint64)
        lsb = (bits >> np.uint64(16)) & np.uint64(1)
        rounded = (bits + np.uint64(0x7FFF) + lsb) >> np.uint64(16)
        out = rounded.astype(np.uint16)
        nan = np.isnan(d)
        if nan.any():
            out[nan] = np.uint16(0x7FC0)
        return out
    raise ValueError(dtype)


def ordered_bits(a, dtype: str) -> np.ndarray:
    """Map stored values to int64 so that consecutive representable numbers differ by 1
    and +0 / -0 coincide."""
    if dtype == "fp32":
        u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.int64)
        sign, mag = u >> 31, u & 0x7FFFFFFF
    elif dtype == "fp16":
        u = np.asarray(a, dtype=np.float16).view(np.uint16).astype(np.int64)
        sign, mag = u >> 15, u & 0x7FFF
    elif dtype == "bf16":
        u = np.asarray(a, dtype=np.uint16).astype(np.int64)
        sign, mag = u >> 15, u & 0x7FFF
    else:
        raise ValueError(dtype)
    return np.where(sign == 1, -mag, mag)


def ulp_distance(a, b, dtype: str) -> np.ndarray:
    """Element-wise distance in units in the last place of the storage type."""
    return np.abs(ordered_bits(a, dtype) - ordered_bits(b, dtype))
