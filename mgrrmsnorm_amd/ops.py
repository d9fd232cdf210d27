"""Tensor-level operators: the one place the Python surface calls into native code.

    rmsnorm_forward(input[R,C], weight[C], epsilon) -> [output, inv_rms(fp32,[R])]
    rmsnorm_backward(grad_output, input, weight, inv_rms) -> [grad_input, grad_weight]

keep the call signatures and return values of the reference's extension module
(pytorch_binding/binding.cpp:16,73-78,136-139); `swiglu_forward` / `swiglu_backward` are the
tensor-level form of its two Triton launches (megagemm/swiglu.py:89-131); `rmsnorm` and
`swiglu` are the differentiable operators the nn.Modules call.

Two bindings of the same C ABI (include/megagemm_hip.h) exist and give identical results:
the compiled torch extension `_binding` (csrc/torch_binding.cpp: checks, allocation and the
autograd nodes in C++), used whenever it has been built, and the ctypes binding
(ops_ctypes.py), which needs no C++ compiler.  Set MGRRMSNORM_BINDING=ctypes before the first
call to force the latter.  There is no CPU path: without the HIP library every call raises.
"""
from __future__ import annotations

import os

import torch

from . import _lib

_binding = None
_resolved = False


def _check_extension_abi(ext) -> None:
    """The extension must have been compiled against this package's header (its own
    MG_ABI_VERSION constant) and must have loaded a library of the same version."""
    built = getattr(ext, "built_abi_version", lambda: None)()
    if built != _lib.ABI_VERSION:
        raise RuntimeError(f"{ext.__file__} was compiled against ABI {built}, "
                           f"this package needs {_lib.ABI_VERSION}; rebuild it")
    if ext.abi_version() != _lib.ABI_VERSION:
        raise RuntimeError(f"{ext.__file__} loaded a libmegagemm_hip.so of ABI {ext.abi_version()}, "
                           f"this package needs {_lib.ABI_VERSION}; rebuild it")


def _extension():
    """The compiled extension module, or None when it is not built / not wanted."""
    global _binding, _resolved
    if _resolved:
        return _binding
    if os.environ.get("MGRRMSNORM_BINDING", "").lower() != "ctypes":
        try:
            from . import _binding as ext

            _check_extension_abi(ext)
            _binding = ext
        except ImportError:
            _binding = None      # not built (or the HIP library is missing: ctypes then says so)
    _resolved = True
    return _binding


def backend() -> str:
    """'extension' when calls go through the compiled torch extension, else 'ctypes'."""
    return "extension" if _extension() is not None else "ctypes"


def rmsnorm_forward(input: torch.Tensor, weight: torch.Tensor, epsilon: float):
    """y = x * rsqrt(mean(x^2) + eps) * w.  Returns [output, inv_rms]."""
    ext = _extension()
    if ext is not None:
        return ext.rmsnorm_forward(input, weight, epsilon)
    from . import ops_ctypes

    return ops_ctypes.rmsnorm_forward(input, weight, epsilon)


def rmsnorm_backward_f32(grad_output, input, weight, inv_rms, need_weight_grad: bool = True):
    """(grad_input, grad_weight fp32, grad_weight in the weight's dtype); the last two are
    None when need_weight_grad is False (the dW reduction is then not launched)."""
    ext = _extension()
    if ext is not None:
        return ext.rmsnorm_backward_f32(grad_output, input, weight, inv_rms, need_weight_grad)
    from . import ops_ctypes

    return ops_ctypes.rmsnorm_backward_f32(grad_output, input, weight, inv_rms, need_weight_grad)


def rmsnorm_backward(grad_output, input, weight, inv_rms):
    """Returns [grad_input, grad_weight]; grad_weight has the weight's dtype
    (binding.cpp:90), rounded once from the fp32 column sums."""
    ext = _extension()
    if ext is not None:
        return ext.rmsnorm_backward(grad_output, input, weight, inv_rms)
    from . import ops_ctypes

    return ops_ctypes.rmsnorm_backward(grad_output, input, weight, inv_rms)


def swiglu_forward(gate_up: torch.Tensor, hidden_dim: int) -> torch.Tensor:
    """gate_up: [M, 2*hidden_dim] = [gate | up] per row -> [M, hidden_dim]."""
    ext = _extension()
    if ext is not None:
        return ext.swiglu_forward(gate_up, hidden_dim)
    from . import ops_ctypes

    return ops_ctypes.swiglu_forward(gate_up, hidden_dim)


def swiglu_backward(grad_out: torch.Tensor, gate_up: torch.Tensor, hidden_dim: int) -> torch.Tensor:
    """grad_out [M, hidden_dim], gate_up [M, 2*hidden_dim] -> [M, 2*hidden_dim] = [d_gate | d_up]."""
    ext = _extension()
    if ext is not None:
        return ext.swiglu_backward(grad_out, gate_up, hidden_dim)
    from . import ops_ctypes

    return ops_ctypes.swiglu_backward(grad_out, gate_up, hidden_dim)


def rmsnorm(input: torch.Tensor, weight: torch.Tensor, epsilon: float = 1e-5) -> torch.Tensor:
    """Differentiable RMSNorm over the last dimension of `input` (any leading dimensions)."""
    ext = _extension()
    if ext is not None:
        return ext.rmsnorm(input, weight, epsilon)     # autograd node in C++
    from .rmsnorm import RMSNormFunction

    if torch.is_grad_enabled() and (input.requires_grad or weight.requires_grad):
        return RMSNormFunction.apply(input, weight, epsilon)
    shape = input.shape
    if len(shape) < 1:
        raise RuntimeError("RMSNorm needs at least one dimension")
    x2d = (input if input.is_contiguous() else input.contiguous()).view(-1, shape[-1])
    w = weight if weight.is_contiguous() else weight.contiguous()
    return rmsnorm_forward(x2d, w, epsilon)[0].view(shape)


def swiglu(w12_out: torch.Tensor, hidden_dim: int) -> torch.Tensor:
    """Differentiable silu(gate) * up over the last dimension of a fused [..., 2*hidden_dim] tensor."""
    ext = _extension()
    if ext is not None:
        return ext.swiglu(w12_out, hidden_dim)         # autograd node in C++
    from .swiglu import MegaGemmFunction

    if torch.is_grad_enabled() and w12_out.requires_grad:
        return MegaGemmFunction.apply(w12_out, hidden_dim)
    if w12_out.dim() < 1 or w12_out.size(-1) != 2 * hidden_dim:
        raise RuntimeError(f"last dimension must be 2*hidden_dim = {2 * hidden_dim}, got {tuple(w12_out.shape)}")
    fused = w12_out if w12_out.is_contiguous() else w12_out.contiguous()
    return swiglu_forward(fused.view(-1, 2 * hidden_dim), hidden_dim).view(*fused.shape[:-1], hidden_dim)
