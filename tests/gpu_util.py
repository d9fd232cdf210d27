"""Helpers for the GPU parity tests: seeded inputs and raw C-ABI calls on torch tensors.
The comparison rules (1e-5 relative for fp32, 1 ulp for fp16/bf16, the counted cancellation
floor for dx and d_gate, the scale-aware dW metric) live in oracle/compare.py.
"""
from __future__ import annotations

import ctypes

import numpy as np
import torch

import oracle
from oracle import compare
from mgrrmsnorm_amd import _lib

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
CODES = {"fp32": 0, "fp16": 1, "bf16": 2}
FP32_ULP = compare.FP32_ULP


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

def assert_matches(got, ref64, dtype, what, floor=None, every_element_cancels=None):
    """compare.assert_matches; a dx of one-column rows (last dimension 1, checked with the dx
    floor) is the all-cancellation case that rule names, wherever a shape list contains it."""
    if every_element_cancels is None:
        every_element_cancels = isinstance(floor, compare.Floor) and got.dim() == 2 and got.shape[-1] == 1
    return compare.assert_matches(got, ref64, dtype, what if not every_element_cancels or "one column" in what
                                  else f"{what} (one column)", floor=floor, every_element_cancels=every_element_cancels)


assert_dw = compare.assert_dw
dx_floor = compare.dx_floor


def rmsnorm_reference(x_cpu, dy_cpu, w_cpu, eps, dtype):
    """Double-precision oracle answers for stored inputs; also the cancellation floor of dx."""
    x32 = oracle.to_f32(as_np(x_cpu, dtype), dtype)
    w32 = oracle.to_f32(as_np(w_cpu, dtype), dtype)
    y, s = oracle.rmsnorm_fwd_f64(x32, w32, eps)
    if dy_cpu is None:
        return y, s, None, None, None
    dy32 = oracle.to_f32(as_np(dy_cpu, dtype), dtype)
    dx, dw = oracle.rmsnorm_bwd_f64(dy32, x32, w32, eps)
    dx32, _ = oracle.rmsnorm_bwd_f32(dy32, x32, w32, s.astype(np.float32))   # the reference's arithmetic
    floor = compare.Floor(dx_floor(x32, dy32, w32, s), dx32)
    return y, s, dx, dw, floor


def swiglu_reference(gu_cpu, dh_cpu, dtype):
    gu32 = oracle.to_f32(as_np(gu_cpu, dtype), dtype)
    h = oracle.swiglu_fwd_f64(gu32)
    if dh_cpu is None:
        return h, None, None
    dh32 = oracle.to_f32(as_np(dh_cpu, dtype), dtype)
    d = oracle.swiglu_bwd_f64(dh32, gu32)
    return h, d, compare.Floor(compare.swiglu_floor(dh32, gu32), oracle.swiglu_bwd_f32(dh32, gu32))
