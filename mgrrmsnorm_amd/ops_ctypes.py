"""Tensor-level operators on top of the C ABI, bound with ctypes: checks, output allocation,
launch.  This is the binding that needs no C++ compiler; `mgrrmsnorm_amd.ops` prefers the
compiled extension (csrc/torch_binding.cpp) over the same C ABI when it has been built and
falls back to this module otherwise.  Both call the same library: there is one kernel path.

`rmsnorm_forward` / `rmsnorm_backward` keep the call signatures and return values of the
reference's extension module (pytorch_binding/binding.cpp:16,73-78,136-139):

    rmsnorm_forward(input[R,C], weight[C], epsilon) -> [output, inv_rms(fp32,[R])]
    rmsnorm_backward(grad_output, input, weight, inv_rms) -> [grad_input, grad_weight]

`swiglu_forward` / `swiglu_backward` are the tensor-level form of the two Triton launches
(megagemm/swiglu.py:89-131).  All four run on torch's current stream of the tensors'
device and never synchronise.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib


def _require_gpu(t: torch.Tensor, name: str) -> None:
    # binding.cpp:9 CHECK_CUDA
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def _require_contiguous(t: torch.Tensor, name: str) -> None:
    # binding.cpp:10 CHECK_CONTIGUOUS
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_pair(input: torch.Tensor, weight: torch.Tensor) -> None:
    if input.dim() != 2:
        raise RuntimeError("Input must be 2D")
    if weight.dim() != 1 or weight.size(0) != input.size(1):
        raise RuntimeError("Weight size must match hidden size")
    if weight.dtype != input.dtype:
        raise RuntimeError(
            f"weight dtype ({weight.dtype}) must equal input dtype ({input.dtype}); "
            "cast the module, e.g. model.half() or model.to(torch.bfloat16)")
    if weight.device != input.device:
        raise RuntimeError("input and weight must be on the same device")


def rmsnorm_forward(input: torch.Tensor, weight: torch.Tensor, epsilon: float):
    """y = x * rsqrt(mean(x^2) + eps) * w.  Returns [output, inv_rms]."""
    if not (input.is_cuda and weight.is_cuda and input.is_contiguous() and weight.is_contiguous()):
        for t, n in ((input, "input"), (weight, "weight")):
            _require_gpu(t, n)
            _require_contiguous(t, n)
    if input.dim() != 2 or weight.dim() != 1 or weight.size(0) != input.size(1) \
            or weight.dtype != input.dtype or weight.device != input.device:
        _check_pair(input, weight)
    code = _lib.dtype_code(input.dtype)
    rows, cols = input.shape
    if cols < 1:
        raise RuntimeError("hidden size must be >= 1")
    lib = _lib.load()
    dev = input.device
    with _lib.device_of(dev):
        output = torch.empty_like(input)
        inv_rms = torch.empty((rows,), dtype=torch.float32, device=dev)
        rc = lib.mg_rmsnorm_fwd(output.data_ptr(), inv_rms.data_ptr(), input.data_ptr(), weight.data_ptr(),
                                rows, cols, epsilon, code, _lib.stream_ptr(dev))
    if rc != 0:
        _lib.check(rc, "RMSNorm forward")
    return [output, inv_rms]


# (device index, rows, cols, dtype code) -> (num_partials, ld); the answer depends on nothing else
# but the tuning options, so the table is dropped whenever the library's count of option changes
# has moved (through _lib.set_option or a direct mg_set_option alike)
_workspace_shapes: dict = {}
_workspace_generation = -1


def _bwd_workspace(lib, dev, rows, cols, code):
    global _workspace_generation
    generation = lib.mg_option_generation()
    if generation != _workspace_generation:
        _workspace_shapes.clear()
        _workspace_generation = generation
    key = (dev.index, rows, cols, code)
    hit = _workspace_shapes.get(key)
    if hit is None:
        n_part, ld = ctypes.c_int64(0), ctypes.c_int64(0)
        _lib.check(lib.mg_rmsnorm_bwd_workspace(rows, cols, code, ctypes.byref(n_part), ctypes.byref(ld)),
                   "RMSNorm backward (workspace query)")
        hit = (n_part.value, ld.value)
        if len(_workspace_shapes) < 4096:
            _workspace_shapes[key] = hit
    return hit


def rmsnorm_backward_f32(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                         inv_rms: torch.Tensor, need_weight_grad: bool = True):
    """Backward with dW kept in fp32: returns (grad_input, grad_weight_f32, grad_weight_cast)
    where grad_weight_cast has the weight's dtype (it is grad_weight_f32 itself for fp32).
    With need_weight_grad=False the dW reduction is not launched and both are None."""
    if not (grad_output.is_cuda and input.is_cuda and weight.is_cuda and inv_rms.is_cuda
            and grad_output.is_contiguous() and input.is_contiguous() and weight.is_contiguous()
            and inv_rms.is_contiguous()):
        for t, n in ((grad_output, "grad_output"), (input, "input"), (weight, "weight"), (inv_rms, "inv_rms")):
            _require_gpu(t, n)
            _require_contiguous(t, n)
    if input.dim() != 2 or weight.dim() != 1 or weight.size(0) != input.size(1) \
            or weight.dtype != input.dtype or weight.device != input.device:
        _check_pair(input, weight)
    if grad_output.shape != input.shape or grad_output.dtype != input.dtype:
        raise RuntimeError("grad_output must have the shape and dtype of input")
    if inv_rms.dtype != torch.float32 or inv_rms.dim() != 1 or inv_rms.size(0) != input.size(0):
        raise RuntimeError("inv_rms must be a float32 vector with one entry per row")
    code = _lib.dtype_code(input.dtype)
    rows, cols = input.shape
    lib = _lib.load()
    dev = input.device
    with _lib.device_of(dev):
        stream = _lib.stream_ptr(dev)
        n_part, ld = _bwd_workspace(lib, dev, rows, cols, code)
        grad_input = torch.empty_like(input)
        partial = torch.empty((n_part, ld), dtype=torch.float32, device=dev)
        dw_f32 = dw_cast = None
        if need_weight_grad:
            dw_f32 = torch.empty((cols,), dtype=torch.float32, device=dev)
            dw_cast = dw_f32 if code == _lib.MG_F32 else torch.empty_like(weight)
        rc = lib.mg_rmsnorm_bwd(grad_input.data_ptr(), partial.data_ptr(), grad_output.data_ptr(),
                                input.data_ptr(), weight.data_ptr(), inv_rms.data_ptr(), rows, cols, code,
                                n_part, ld, stream)
        if rc != 0:
            _lib.check(rc, "RMSNorm backward")
        if need_weight_grad:
            rc = lib.mg_rmsnorm_dw_reduce(dw_f32.data_ptr(), None if dw_cast is dw_f32 else dw_cast.data_ptr(),
                                          code, partial.data_ptr(), n_part, ld, cols, stream)
            if rc != 0:
                _lib.check(rc, "RMSNorm backward (dW reduction)")
    return grad_input, dw_f32, dw_cast


def rmsnorm_backward(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                     inv_rms: torch.Tensor):
    """Returns [grad_input, grad_weight]; grad_weight has the weight's dtype
    (binding.cpp:90), rounded once from the fp32 column sums."""
    grad_input, _, dw_cast = rmsnorm_backward_f32(grad_output, input, weight, inv_rms)
    return [grad_input, dw_cast]


def swiglu_forward(gate_up: torch.Tensor, hidden_dim: int) -> torch.Tensor:
    """gate_up: [M, 2*hidden_dim] = [gate | up] per row -> [M, hidden_dim]."""
    _require_gpu(gate_up, "w12_out")
    _require_contiguous(gate_up, "w12_out")
    if gate_up.dim() != 2 or gate_up.size(1) != 2 * hidden_dim:
        raise RuntimeError(f"expected a [M, {2 * hidden_dim}] matrix, got {tuple(gate_up.shape)}")
    code = _lib.dtype_code(gate_up.dtype)
    M = gate_up.size(0)
    lib = _lib.load()
    with _lib.device_of(gate_up.device):
        out = torch.empty((M, hidden_dim), dtype=gate_up.dtype, device=gate_up.device)
        rc = lib.mg_swiglu_fwd(out.data_ptr(), gate_up.data_ptr(), M, hidden_dim, code,
                               _lib.stream_ptr(gate_up.device))
    _lib.check(rc, "SwiGLU forward")
    return out


def swiglu_backward(grad_out: torch.Tensor, gate_up: torch.Tensor, hidden_dim: int) -> torch.Tensor:
    """grad_out: [M, hidden_dim], gate_up: [M, 2*hidden_dim] -> [M, 2*hidden_dim] = [d_gate | d_up]."""
    for t, n in ((grad_out, "grad_output"), (gate_up, "w12_out")):
        _require_gpu(t, n)
        _require_contiguous(t, n)
    if gate_up.dim() != 2 or gate_up.size(1) != 2 * hidden_dim:
        raise RuntimeError(f"expected a [M, {2 * hidden_dim}] matrix, got {tuple(gate_up.shape)}")
    if grad_out.shape != (gate_up.size(0), hidden_dim) or grad_out.dtype != gate_up.dtype:
        raise RuntimeError("grad_output must be [M, hidden_dim] with the dtype of the forward input")
    code = _lib.dtype_code(gate_up.dtype)
    M = gate_up.size(0)
    lib = _lib.load()
    with _lib.device_of(gate_up.device):
        grad_in = torch.empty_like(gate_up)
        rc = lib.mg_swiglu_bwd(grad_in.data_ptr(), grad_out.data_ptr(), gate_up.data_ptr(), M, hidden_dim, code,
                               _lib.stream_ptr(gate_up.device))
    _lib.check(rc, "SwiGLU backward")
    return grad_in
