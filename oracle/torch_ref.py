"""The reference's PyTorch formulations of the path, restated with stock torch ops.

TEST / BASELINE INFRASTRUCTURE ONLY (same rule as the rest of oracle/): used by tests as a
second opinion and by bench.py's cpu_baseline leg, where it is the thing timed on the host
cores.  Never imported by the product.

  rmsnorm_formula   test_rmsnorm.py:55-56 and colab_test.py:176
  swiglu_formula    benchmark_swiglu.py:57 on the fused [gate | up] layout of megagemm/swiglu.py:35-36
"""
import torch
import torch.nn.functional as F


def rmsnorm_formula(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def rmsnorm_fwd_bwd(x: torch.Tensor, w: torch.Tensor, dy: torch.Tensor, eps: float):
    """Forward and autograd backward with loss = sum(y * dy). Returns (y, dx, dW)."""
    x = x.detach().requires_grad_(True)
    w = w.detach().requires_grad_(True)
    y = rmsnorm_formula(x, w, eps)
    (y * dy).sum().backward()
    return y.detach(), x.grad, w.grad


def swiglu_formula(gu: torch.Tensor) -> torch.Tensor:
    H = gu.shape[-1] // 2
    return F.silu(gu[..., :H]) * gu[..., H:]


def swiglu_fwd_bwd(gu: torch.Tensor, dh: torch.Tensor):
    gu = gu.detach().requires_grad_(True)
    h = swiglu_formula(gu)
    (h * dh).sum().backward()
    return h.detach(), gu.grad
