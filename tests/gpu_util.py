"""Helpers for the GPU parity tests: seeded inputs, raw C-ABI calls on torch tensors, and
the comparison rules.

Comparison rules (from the build's stated tolerances):
  fp32 outputs       |got - ref| <= 1e-5 * |ref|  (+ the cancellation floor below)
  fp16/bf16 outputs  at most 1 unit in the last place away from the double-precision
                     oracle rounded once to the output type
  cancellation floor dx and d_gate are sums of terms of either sign:
                       dx[r,c] = s*dy*w  -  sum_j x[r,c]*(s^3/C)*dy[r,j]*w[j]*x[r,j]
                     Where the terms nearly cancel, no fp32 evaluation (the reference's
                     included) resolves the result to 1 ulp of itself; what fp32 arithmetic
                     does guarantee is the forward error bound of a computed sum, a few ulps
                     of the sum of the terms' magnitudes.  An element therefore also passes
                     when |got - ref| <= 8 * 2^-24 * (sum of |terms|).
  dW                 on the fp32 buffer, scale-aware: max|got - ref| / max|ref| <= 1e-3 and
                     ||got - ref||_2 / ||ref||_2 <= 1e-3; bit-identical from run to run.
"""
from __future__ import annotations

import ctypes

import numpy as np
import torch

import oracle
from mgrrmsnorm_amd import _lib

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
CODES = {"fp32": 0, "fp16": 1, "bf16": 2}
FP32_ULP = 2.0 ** -24


def lib():
    return _lib.load()


def stream():
    return torch.cuda.current_stream().cuda_stream


def check(rc, what="call"):
    assert rc == 0, f"{what} failed with {rc}: {lib().mg_last_error().decode()}"


# ------------------------------------------------------------------------------- inputs

def cpu_randn(shape, seed, outliers=False):
    """fp32 N(0,1) from a seeded CPU generator; with `outliers`, an independent 1% of the
    entries is multiplied by 100."""
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(shape, generator=g, dtype=torch.float32)
    if outliers:
        mask = torch.rand(shape, generator=g) < 0.01
        t = torch.where(mask, t * 100.0, t)
    return t


def rmsnorm_inputs(rows, cols, dtype, seed=42, outliers=False):
    """x, dy ~ N(0,1), w = 1 + 0.02 N(0,1), generated in fp32 on the CPU, then rounded to
    the storage type.  Returns torch CPU tensors of that type."""
    td = DTYPES[dtype]
    x = cpu_randn((rows, cols), seed, outliers).to(td)
    dy = cpu_randn((rows, cols), seed + 1000, outliers).to(td)
    w = (1.0 + 0.02 * cpu_randn((cols,), seed + 2000)).to(td)
    return x, dy, w


def as_np(t: torch.Tensor, dtype: str) -> np.ndarray:
    """Storage-type view for the oracle helpers: float32 / float16 arrays, uint16 bits for bf16."""
    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def as_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().float().numpy()


# ------------------------------------------------------------------------ raw ABI calls

def rmsnorm_fwd(x: torch.Tensor, w: torch.Tensor, eps: float, dtype: str, want_inv_rms=True):
    rows, cols = x.shape
    y = torch.empty_like(x)
    s = torch.empty(rows, dtype=torch.float32, device=x.device) if want_inv_rms else None
    check(lib().mg_rmsnorm_fwd(y.data_ptr(), s.data_ptr() if want_inv_rms else None, x.data_ptr(), w.data_ptr(),
                               rows, cols, eps, CODES[dtype], stream()), "mg_rmsnorm_fwd")
    return y, s


def bwd_workspace(rows, cols, dtype):
    P, ld = ctypes.c_int64(0), ctypes.c_int64(0)
    check(lib().mg_rmsnorm_bwd_workspace(rows, cols, CODES[dtype], ctypes.byref(P), ctypes.byref(ld)),
          "mg_rmsnorm_bwd_workspace")
    return P.value, ld.value


def rmsnorm_bwd(dy, x, w, s, dtype, num_partials=None, want_cast=True):
    rows, cols = x.shape
    P, ld = bwd_workspace(rows, cols, dtype)
    if num_partials is not None:
        P = num_partials
    dx = torch.empty_like(x)
    part = torch.full((P, ld), float("nan"), dtype=torch.float32, device=x.device)
    check(lib().mg_rmsnorm_bwd(dx.data_ptr(), part.data_ptr(), dy.data_ptr(), x.data_ptr(), w.data_ptr(),
                               s.data_ptr(), rows, cols, CODES[dtype], P, ld, stream()), "mg_rmsnorm_bwd")
    dw = torch.empty(cols, dtype=torch.float32, device=x.device)
    dwc = torch.empty_like(w) if want_cast else None
    check(lib().mg_rmsnorm_dw_reduce(dw.data_ptr(), dwc.data_ptr() if want_cast else None, CODES[dtype],
                                     part.data_ptr(), P, ld, cols, stream()), "mg_rmsnorm_dw_reduce")
    return dx, dw, dwc, part


def swiglu_fwd(gu: torch.Tensor, H: int, dtype: str):
    M = gu.shape[0]
    h = torch.empty((M, H), dtype=gu.dtype, device=gu.device)
    check(lib().mg_swiglu_fwd(h.data_ptr(), gu.data_ptr(), M, H, CODES[dtype], stream()), "mg_swiglu_fwd")
    return h


def swiglu_bwd(dh: torch.Tensor, gu: torch.Tensor, H: int, dtype: str):
    M = gu.shape[0]
    dgu = torch.empty_like(gu)
    check(lib().mg_swiglu_bwd(dgu.data_ptr(), dh.data_ptr(), gu.data_ptr(), M, H, CODES[dtype], stream()),
          "mg_swiglu_bwd")
    return dgu


# -------------------------------------------------------------------------- comparisons

def assert_matches(got: torch.Tensor, ref64: np.ndarray, dtype: str, what: str, floor: np.ndarray | None = None):
    """Apply the output rule of this module's docstring to one tensor."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    g_store = as_np(got, dtype)
    g64 = oracle.to_f32(g_store, dtype).astype(np.float64)
    assert g64.shape == ref64.shape, f"{what}: shape {g64.shape} vs {ref64.shape}"
    assert np.isfinite(g64).all(), f"{what}: non-finite values in the output"
    err = np.abs(g64 - ref64)
    if dtype == "fp32":
        bad = err > 1e-5 * np.abs(ref64) + 1e-37
        detail = lambda i: f"rel err {err[i] / max(abs(ref64[i]), 1e-300):.3e}"
    else:
        ulps = oracle.ulp_distance(g_store, oracle.round_to(ref64, dtype), dtype)
        bad = ulps > 1
        detail = lambda i: f"{ulps[i]} ulp"
    if floor is not None:
        bad &= err > 8 * FP32_ULP * floor
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, err, -1.0)), err.shape)
        raise AssertionError(
            f"{what} [{dtype}]: {int(bad.sum())} of {bad.size} elements out of tolerance; worst at {idx}: "
            f"got {g64[idx]!r}, ref {ref64[idx]!r}, {detail(idx)}")


def assert_dw(dw_f32: torch.Tensor, ref64: np.ndarray, what="dW"):
    got = dw_f32.detach().cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite"
    scale = max(np.abs(ref64).max(), 1e-300)
    e_max = np.abs(got - ref64).max() / scale
    e_l2 = np.linalg.norm(got - ref64) / max(np.linalg.norm(ref64), 1e-300)
    assert e_max <= 1e-3 and e_l2 <= 1e-3, f"{what}: max-scaled err {e_max:.3e}, l2 err {e_l2:.3e}"
    return e_max, e_l2


def dx_floor(x, dy, w, s):
    """Sum of the magnitudes of the terms dx is made of (see the module docstring)."""
    x, dy, w, s = (np.asarray(a, dtype=np.float64) for a in (x, dy, w, s))
    cols = x.shape[1]
    gwx = np.abs(dy * w * x).sum(-1, keepdims=True)
    return np.abs(s[:, None] * dy * w) + np.abs(x) * (s[:, None] ** 3 / cols) * gwx


def rmsnorm_reference(x_cpu, dy_cpu, w_cpu, eps, dtype):
    """Double-precision oracle answers for stored inputs; also the cancellation floor of dx."""
    x32 = oracle.to_f32(as_np(x_cpu, dtype), dtype)
    w32 = oracle.to_f32(as_np(w_cpu, dtype), dtype)
    y, s = oracle.rmsnorm_fwd_f64(x32, w32, eps)
    if dy_cpu is None:
        return y, s, None, None, None
    dy32 = oracle.to_f32(as_np(dy_cpu, dtype), dtype)
    dx, dw = oracle.rmsnorm_bwd_f64(dy32, x32, w32, eps)
    floor = dx_floor(x32, dy32, w32, s)
    return y, s, dx, dw, floor


def swiglu_reference(gu_cpu, dh_cpu, dtype):
    gu32 = oracle.to_f32(as_np(gu_cpu, dtype), dtype)
    h = oracle.swiglu_fwd_f64(gu32)
    if dh_cpu is None:
        return h, None, None
    dh32 = oracle.to_f32(as_np(dh_cpu, dtype), dtype)
    d = oracle.swiglu_bwd_f64(dh32, gu32)
    H = gu32.shape[1] // 2
    g, u = gu32[:, :H].astype(np.float64), gu32[:, H:].astype(np.float64)
    sig = 1.0 / (1.0 + np.exp(-g))
    base = np.abs(dh32.astype(np.float64) * u * sig)
    floor = np.concatenate([base * (1.0 + np.abs(g) * (1.0 - sig)), np.zeros_like(base)], axis=1)
    return h, d, floor
