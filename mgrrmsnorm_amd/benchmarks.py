"""Comparison benchmarks in the style of the reference's scripts: stock PyTorch against
this package, wall-clock per call with a device synchronisation on both sides.

    python -m mgrrmsnorm_amd.benchmarks swiglu     # benchmark_swiglu.py:61-181 (block forward, 3 configs)
    python -m mgrrmsnorm_amd.benchmarks rmsnorm    # colab_test.py:143-184 / README.md:28-35: forward and
                                                   # forward+backward, fp16 and bf16
    python -m mgrrmsnorm_amd.benchmarks all

Method as in the reference (benchmark_swiglu.py:16-37): 10 warm-up calls, then 100 calls each
bracketed by torch.cuda.synchronize() and time.perf_counter(); mean and standard deviation
in milliseconds, speed-up of this package over PyTorch, peak device memory.  A call of 13-35 us
of GPU work timed that way is mostly the latency of one launch and one synchronisation, the
same for every implementation, so the RMSNorm tables carry a second column: GPU time per call,
from device events around the same calls issued back to back.  For kernel-level bandwidth
figures use bench.py at the repository root instead.
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


def gpu_time_per_call(fn, warmup: int = 10, iterations: int = 100):
    """GPU time of fn() in milliseconds: device events around `iterations` calls issued back to
    back (no synchronisation in between), best of three."""
    for _ in range(warmup):
        fn()
    best = None
    for _ in range(3):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(iterations):
            fn()
        b.record()
        b.synchronize()
        t = a.elapsed_time(b) / iterations
        best = t if best is None else min(best, t)
    return best


def _report(title, rows):
    """rows: (name, mean ms, std ms[, GPU ms per call])."""
    with_gpu = len(rows[0]) > 3
    width = 84 if with_gpu else 64
    print(f"\n{'=' * width}\n{title}\n{'=' * width}")
    print(f"{'Implementation':<26}{'Time (ms)':<22}{'Speedup':>10}" + (f"{'GPU time (ms)':>16}{'':>4}" if with_gpu else ""))
    print("-" * width)
    base = rows[0][1]
    for row in rows:
        name, mean, std = row[:3]
        line = f"{name:<26}{mean:>8.3f} +/- {std:<8.3f}{base / mean:>12.2f}x"
        if with_gpu:
            line += f"{row[3]:>14.4f} {rows[0][3] / row[3]:>5.2f}x"
        print(line)
    print("=" * width)


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


def bench_rmsnorm(dtype=torch.float16, configs=None, warmup: int = 10, iterations: int = 100, backward: bool = False):
    """Forward (or forward + backward), PyTorch formula and torch.nn.RMSNorm against this package;
    returns {(batch, seq, hidden): {"formula_ms", "native_ms", "hip_ms": (mean, std), "formula_gpu_ms",
    "native_gpu_ms", "hip_gpu_ms": float, "max_diff": float}}."""
    results = {}
    for batch, seq, hidden in (RMSNORM_CONFIGS if configs is None else configs):
        x = torch.randn(batch, seq, hidden, device="cuda", dtype=dtype, requires_grad=backward)
        dy = torch.randn(batch, seq, hidden, device="cuda", dtype=dtype)
        ours = RMSNorm(hidden, 1e-6).cuda().to(dtype)
        native = torch.nn.RMSNorm(hidden, eps=1e-6).cuda().to(dtype)
        w = ours.weight if backward else ours.weight.detach()

        def formula():                               # colab_test.py:176
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

        def run(f):
            if not backward:
                return lambda: f()

            def step():
                x.grad = None
                ours.weight.grad = None
                native.weight.grad = None
                f().backward(dy)
            return step

        calls = [("PyTorch formula", run(formula)), ("torch.nn.RMSNorm", run(lambda: native(x))),
                 ("mgrrmsnorm_amd (HIP)", run(lambda: ours(x)))]
        import contextlib

        with (contextlib.nullcontext() if backward else torch.no_grad()):
            wall = [time_calls(f, warmup, iterations) for _, f in calls]
            gpu = [gpu_time_per_call(f, warmup, iterations) for _, f in calls]
        with torch.no_grad():
            diff = (formula().float() - ours(x).float()).abs().max().item()
        what = "forward + backward" if backward else "forward"
        _report(f"RMSNorm {what}  batch={batch} seq={seq} hidden={hidden} {dtype}",
                [(name, *wall[i], gpu[i]) for i, (name, _) in enumerate(calls)])
        tokens = batch * seq
        print(f"tokens per second: PyTorch formula {tokens / wall[0][0] * 1e3:,.0f}, "
              f"this package {tokens / wall[2][0] * 1e3:,.0f}")
        print(f"max |difference| vs the formula = {diff:.6f}")
        results[(batch, seq, hidden)] = {"formula_ms": wall[0], "native_ms": wall[1], "hip_ms": wall[2],
                                         "formula_gpu_ms": gpu[0], "native_gpu_ms": gpu[1], "hip_gpu_ms": gpu[2],
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
        for dtype in (torch.float16, torch.bfloat16):
            bench_rmsnorm(dtype=dtype)
            bench_rmsnorm(dtype=dtype, backward=True)
    if what in ("swiglu", "all"):
        bench_swiglu()


if __name__ == "__main__":
    main()
