"""Comparison benchmarks in the style of the reference's scripts: stock PyTorch against
this package, wall-clock per call with a device synchronisation on both sides.

    python -m mgrrmsnorm_amd.benchmarks swiglu     # benchmark_swiglu.py:61-181 (block forward, 3 configs)
    python -m mgrrmsnorm_amd.benchmarks rmsnorm    # colab_test.py:143-184 / README.md:28-35 (fp16 forward)
    python -m mgrrmsnorm_amd.benchmarks all

Method as in the reference (benchmark_swiglu.py:16-37): 10 warm-up calls, then 100 calls each
bracketed by torch.cuda.synchronize() and time.perf_counter(); mean and standard deviation
in milliseconds, speed-up of this package over PyTorch, peak device memory.  For kernel-level
bandwidth figures use bench.py at the repository root instead.
"""
from __future__ import annotations

import sys
import time

import torch
import torch.nn.functional as F

from . import MegaGemmTriton, RMSNorm

SWIGLU_CONFIGS = [(8, 128, 2048), (16, 256, 4096), (32, 512, 4096)]   # benchmark_swiglu.py:167-172
RMSNORM_CONFIGS = [(32, 128, 4096)]                                    # README.md:32,35


def time_calls(fn, warmup: int = 10, iterations: int = 100):
    """Mean and standard deviation of the wall time of fn() in milliseconds."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    samples = []
    for _ in range(iterations):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        samples.append((time.perf_counter() - t0) * 1e3)
    mean = sum(samples) / len(samples)
    var = sum((s - mean) ** 2 for s in samples) / len(samples)
    return mean, var ** 0.5


class UnfusedSwiGLU(torch.nn.Module):
    """The PyTorch baseline: separate gate and up projections, F.silu, down projection
    (benchmark_swiglu.py:40-58)."""

    def __init__(self, d_model: int, hidden: int):
        super().__init__()
        self.w1 = torch.nn.Linear(d_model, hidden, bias=False)
        self.w2 = torch.nn.Linear(d_model, hidden, bias=False)
        self.w3 = torch.nn.Linear(hidden, d_model, bias=False)

    def forward(self, x):
        return self.w3(F.silu(self.w1(x)) * self.w2(x))


def _report(title, rows):
    print(f"\n{'=' * 64}\n{title}\n{'=' * 64}")
    print(f"{'Implementation':<26}{'Time (ms)':<22}{'Speedup':>10}")
    print("-" * 64)
    base = rows[0][1]
    for name, mean, std in rows:
        print(f"{name:<26}{mean:>8.3f} +/- {std:<8.3f}{base / mean:>12.2f}x")
    print("=" * 64)


def bench_swiglu(dtype=torch.float16, configs=None, warmup: int = 10, iterations: int = 100):
    """Block forward, PyTorch baseline against this package with the same weights; returns
    {(batch, seq, d_model): {"pytorch_ms": (mean, std), "hip_ms": (mean, std), "max_diff": float}}."""
    results = {}
    for batch, seq, d_model in (SWIGLU_CONFIGS if configs is None else configs):
        torch.cuda.reset_peak_memory_stats()
        x = torch.randn(batch, seq, d_model, device="cuda", dtype=dtype)
        ours = MegaGemmTriton(d_model).cuda().to(dtype)
        base = UnfusedSwiGLU(d_model, ours.hidden).cuda().to(dtype)
        with torch.no_grad():                       # same weights on both sides (benchmark_swiglu.py:85-89)
            ours.w12.weight[: ours.hidden] = base.w1.weight
            ours.w12.weight[ours.hidden:] = base.w2.weight
            ours.w3.weight.copy_(base.w3.weight)
            t_base = time_calls(lambda: base(x), warmup, iterations)
            t_ours = time_calls(lambda: ours(x), warmup, iterations)
            diff = (base(x) - ours(x)).abs().max().item()
        _report(f"SwiGLU block forward  batch={batch} seq={seq} d_model={d_model} hidden={ours.hidden} {dtype}",
                [("PyTorch native", *t_base), ("mgrrmsnorm_amd (HIP)", *t_ours)])
        print(f"max |difference| = {diff:.6f} ({'ok' if diff < 1e-2 else 'LARGE'}; the reference accepts < 1e-2)")
        print(f"peak memory: allocated {torch.cuda.max_memory_allocated() / 1e9:.2f} GB, "
              f"reserved {torch.cuda.max_memory_reserved() / 1e9:.2f} GB")
        results[(batch, seq, d_model)] = {"pytorch_ms": t_base, "hip_ms": t_ours, "max_diff": diff}
        del x, ours, base
        torch.cuda.empty_cache()
    return results


def bench_rmsnorm(dtype=torch.float16, configs=None, warmup: int = 10, iterations: int = 100):
    """Forward, PyTorch formula and torch.nn.RMSNorm against this package; returns
    {(batch, seq, hidden): {"formula_ms", "native_ms", "hip_ms": (mean, std), "max_diff": float}}."""
    results = {}
    for batch, seq, hidden in (RMSNORM_CONFIGS if configs is None else configs):
        x = torch.randn(batch, seq, hidden, device="cuda", dtype=dtype)
        ours = RMSNorm(hidden, 1e-6).cuda().to(dtype)
        native = torch.nn.RMSNorm(hidden, eps=1e-6).cuda().to(dtype)
        w = ours.weight.detach()

        def formula():                               # colab_test.py:176
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

        with torch.no_grad():
            t_formula = time_calls(formula, warmup, iterations)
            t_native = time_calls(lambda: native(x), warmup, iterations)
            t_ours = time_calls(lambda: ours(x), warmup, iterations)
            diff = (formula().float() - ours(x).float()).abs().max().item()
        _report(f"RMSNorm forward  batch={batch} seq={seq} hidden={hidden} {dtype}",
                [("PyTorch formula", *t_formula), ("torch.nn.RMSNorm", *t_native), ("mgrrmsnorm_amd (HIP)", *t_ours)])
        tokens = batch * seq
        print(f"tokens per second: PyTorch formula {tokens / t_formula[0] * 1e3:,.0f}, "
              f"this package {tokens / t_ours[0] * 1e3:,.0f}")
        print(f"max |difference| vs the formula = {diff:.6f}")
        results[(batch, seq, hidden)] = {"formula_ms": t_formula, "native_ms": t_native, "hip_ms": t_ours,
                                         "max_diff": diff}
    return results


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    what = argv[0] if argv else "all"
    if what not in ("swiglu", "rmsnorm", "all"):
        raise SystemExit(__doc__)
    if not torch.cuda.is_available():
        raise SystemExit("no GPU visible")
    print(f"GPU: {torch.cuda.get_device_name()}   PyTorch: {torch.__version__}")
    if what in ("rmsnorm", "all"):
        bench_rmsnorm()
    if what in ("swiglu", "all"):
        bench_swiglu()


if __name__ == "__main__":
    main()
