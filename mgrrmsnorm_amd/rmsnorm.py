"""RMSNorm for MI355X: autograd function and nn.Module with the reference's surface.

Same names, argument order, defaults, parameter name and repr as the reference's
megagemm/rmsnorm.py:18-78 (`RMSNormFunction.apply(input, weight, epsilon=1e-5)`,
`RMSNorm(hidden_size, epsilon=1e-5)` with a `weight` parameter of ones), so a state_dict or a
call site written for the reference works unchanged.  The arithmetic runs in hand-written
HIP kernels reached through mgrrmsnorm_amd.ops; there is no other code path.  `RMSNorm` calls
the operator's C++ autograd node when the compiled extension is present (no Python in
backward); `RMSNormFunction` is the same flow as a Python autograd.Function.
"""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable

from . import ops


class RMSNormFunction(torch.autograd.Function):
    """y = x * rsqrt(mean(x^2, -1) + epsilon) * weight over the last dimension.

    forward saves (x as [rows, C], weight, inv_rms[rows] fp32) like the reference
    (megagemm/rmsnorm.py:32); backward returns (dx, dW, None) with dW in weight's dtype,
    summed in fp32 in a fixed order (the reference adds per-block partials with atomics,
    src/rmsnorm_kernel.cu:315-325).
    """

    @staticmethod
    def forward(ctx, input: torch.Tensor, weight: torch.Tensor, epsilon: float = 1e-5):
        shape = input.shape
        if len(shape) < 1:
            raise RuntimeError("RMSNorm needs at least one dimension")
        x2d = (input if input.is_contiguous() else input.contiguous()).view(-1, shape[-1])
        w = weight if weight.is_contiguous() else weight.contiguous()
        y2d, inv_rms = ops.rmsnorm_forward(x2d, w, epsilon)
        ctx.save_for_backward(x2d, w, inv_rms)
        ctx.epsilon = epsilon
        ctx.orig_shape = shape
        return y2d.view(shape)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output: torch.Tensor):
        x2d, w, inv_rms = ctx.saved_tensors
        dy2d = (grad_output if grad_output.is_contiguous() else grad_output.contiguous()).view(x2d.shape)
        if dy2d.dtype != x2d.dtype:
            dy2d = dy2d.to(x2d.dtype)
        dx2d, _, dw = ops.rmsnorm_backward_f32(dy2d, x2d, w, inv_rms, need_weight_grad=ctx.needs_input_grad[1])
        return dx2d.view(ctx.orig_shape), dw, None


class RMSNorm(nn.Module):
    """Root-mean-square layer normalisation over the last dimension, on MI355X.

    Args:
        hidden_size: size of the last dimension.
        epsilon: added to the mean square before the reciprocal square root (default 1e-5).

    The compute type follows the input (float32, float16 or bfloat16; accumulation is
    always float32) and the weight must have the input's dtype: cast the module with
    `.half()` / `.to(torch.bfloat16)` as with the reference.
    """

    def __init__(self, hidden_size: int, epsilon: float = 1e-5, *, eps: float | None = None):
        super().__init__()
        if eps is not None:  # torch.nn.RMSNorm spelling, accepted as an alias
            epsilon = eps
        self.hidden_size = hidden_size
        self.epsilon = epsilon
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        # one call: the compiled extension holds the autograd node (same flow as
        # RMSNormFunction, in C++); without it ops.rmsnorm goes through RMSNormFunction.
        # Nothing to differentiate (inference, torch.no_grad()): same kernel, no node.
        return ops.rmsnorm(input, self.weight, self.epsilon)

    def extra_repr(self) -> str:
        return f"hidden_size={self.hidden_size}, eps={self.epsilon}"
