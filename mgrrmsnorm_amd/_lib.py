"""ctypes binding of libmegagemm_hip.so (the C ABI declared in include/megagemm_hip.h).

Together with the compiled extension `_binding` (csrc/torch_binding.cpp, preferred by
mgrrmsnorm_amd.ops when it is built) this takes the place of the reference's pybind11
extension module `rmsnorm_cuda_ops` (pytorch_binding/binding.cpp) and of the Triton launch
sites in megagemm/swiglu.py:100-107,122-129.  The tuning and measurement entry points
(include/megagemm_hip_tuning.h) are reachable through this module only.

There is no CPU fallback: if the library is missing or a call fails, a RuntimeError is
raised with the library's own message.
"""
from __future__ import annotations

import ctypes
import threading
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "libmegagemm_hip.so"
ABI_VERSION = 2

MG_F32, MG_F16, MG_BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: MG_F32, torch.float16: MG_F16, torch.bfloat16: MG_BF16}

_lock = threading.Lock()
_lib = None

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int

# name -> (restype, argtypes); mirrors include/megagemm_hip.h and megagemm_hip_tuning.h one to one
SIGNATURES = {
    "mg_abi_version": (_int, []),
    "mg_last_error": (ctypes.c_char_p, []),
    "mg_set_option": (_int, [ctypes.c_char_p, _int]),
    "mg_option_generation": (_int, []),
    "mg_rmsnorm_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_float, _int, _vp]),
    "mg_rmsnorm_bwd_workspace": (_int, [_i64, _i64, _int, ctypes.POINTER(_i64), ctypes.POINTER(_i64)]),
    "mg_rmsnorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _i64, _i64, _vp]),
    "mg_rmsnorm_dw_reduce": (_int, [_vp, _vp, _int, _vp, _i64, _i64, _i64, _vp]),
    "mg_rmsnorm_bwd_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "mg_swiglu_fwd": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "mg_swiglu_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "mg_copy_bytes": (_int, [_vp, _vp, _i64, _vp]),
    "mg_stream_probe": (_int, [_vp, _vp, _vp, _i64, _vp]),
    "mg_row_probe": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mg_rmsnorm_launch_info": (_int, [_int, _i64, _int] + [ctypes.POINTER(_int)] * 4),
    "mg_rmsnorm_bwd_timeline": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _i64, _i64, _vp, _vp]),
}


def load() -> ctypes.CDLL:
    """Load the library once per process; raise RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"HIP library not built: {LIB_PATH} is missing. "
                "Run: python -m mgrrmsnorm_amd._build   (needs hipcc; builds for gfx950)")
        try:
            lib = ctypes.CDLL(str(LIB_PATH))
        except OSError as exc:  # e.g. libamdhip64.so not found
            raise RuntimeError(f"cannot load {LIB_PATH}: {exc}") from exc
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.mg_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}; rebuild it")
        _lib = lib
    return _lib


def last_error() -> str:
    return load().mg_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed (code {rc}): {last_error()}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError(
            f"Unsupported dtype {dtype}. Use float32, float16, or bfloat16.") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """Raw hipStream_t of torch's current stream on `device`."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)     # no Stream object is built on this path
    return torch.cuda.current_stream(device).cuda_stream


class device_of:
    """Makes the tensor's device current for the enclosed launches, like
    torch.cuda.device(...) but free when it already is (the common case)."""

    __slots__ = ("idx", "prev")

    def __init__(self, device: torch.device):
        self.idx = device.index
        self.prev = -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)
        return self

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


def set_option(key: str, value: int) -> None:
    """Tuning hook (mg_set_option).  The workspace shapes the ctypes binding remembers follow
    the library's own count of option changes, so nothing has to be cleared here."""
    check(load().mg_set_option(key.encode(), int(value)), "mg_set_option")
