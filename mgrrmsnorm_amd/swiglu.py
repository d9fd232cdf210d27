"""SwiGLU block for MI355X: fused-activation autograd function and the nn.Module.

Keeps the surface of the reference's megagemm/swiglu.py:86-172:
`MegaGemmFunction.apply(w12_out, hidden_dim)` maps [..., 2*hidden] = [gate | up] to
[..., hidden] = silu(gate) * up, and `MegaGemmTriton(d_model, multiple_of=256,
hidden_multiple=5/3)` owns `w12` (d_model -> 2*hidden) and `w3` (hidden -> d_model), both
bias-free nn.Linear layers that stay on torch.matmul.  The class keeps its historical name
for drop-in use; nothing here uses Triton -- the activation and its backward are HIP
kernels reached through mgrrmsnorm_amd.ops.
"""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable

from . import ops


class MegaGemmFunction(torch.autograd.Function):
    """silu(gate) * up on a fused [..., 2*hidden_dim] tensor, reading both halves in place."""

    @staticmethod
    def forward(ctx, w12_out: torch.Tensor, hidden_dim: int):
        if w12_out.size(-1) != 2 * hidden_dim:
            raise RuntimeError(
                f"last dimension must be 2*hidden_dim = {2 * hidden_dim}, got {w12_out.size(-1)}")
        fused = w12_out.contiguous()
        ctx.save_for_backward(fused)
        ctx.hidden_dim = hidden_dim
        out = ops.swiglu_forward(fused.view(-1, 2 * hidden_dim), hidden_dim)
        return out.view(*fused.shape[:-1], hidden_dim)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output: torch.Tensor):
        (fused,) = ctx.saved_tensors
        hidden_dim = ctx.hidden_dim
        dh = grad_output.contiguous().view(-1, hidden_dim)
        if dh.dtype != fused.dtype:
            dh = dh.to(fused.dtype)
        grad = ops.swiglu_backward(dh, fused.view(-1, 2 * hidden_dim), hidden_dim)
        return grad.view(fused.shape), None


class MegaGemmTriton(nn.Module):
    """SwiGLU feed-forward block: w3(silu(w1 x) * (w2 x)) with w1 and w2 fused into w12.

    Args:
        d_model: input and output width.
        multiple_of: the hidden width is rounded up to a multiple of this (default 256).
        hidden_multiple: expansion factor before rounding (default 5/3).

    Rows [0, hidden) of `w12.weight` are the gate projection and rows [hidden, 2*hidden)
    the up projection, as in the reference (benchmark_swiglu.py:87-88).
    """

    def __init__(self, d_model: int, multiple_of: int = 256, hidden_multiple: float = 5 / 3):
        super().__init__()
        raw = int(d_model * hidden_multiple)
        self.hidden = multiple_of * ((raw + multiple_of - 1) // multiple_of)
        self.w12 = nn.Linear(d_model, 2 * self.hidden, bias=False)
        self.w3 = nn.Linear(self.hidden, d_model, bias=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # the activation's autograd node lives in the compiled extension when that is built
        # (else MegaGemmFunction); with nothing to differentiate it is the bare kernel
        return self.w3(ops.swiglu(self.w12(x), self.hidden))

    def extra_repr(self) -> str:
        return f"d_model={self.w12.in_features}, hidden={self.hidden} (Triton Accelerated)"
