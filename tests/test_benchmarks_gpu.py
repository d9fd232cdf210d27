"""The comparison harness (mgrrmsnorm_amd/benchmarks.py, after the reference's
benchmark_swiglu.py:61-155 and colab_test.py:143-184) on one small configuration each: the
result structure, and the reference's own acceptance check -- block output within 1e-2 of
the unfused PyTorch block with the same weights (benchmark_swiglu.py:117-129)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_swiglu_block_benchmark(capsys):
    from mgrrmsnorm_amd import benchmarks

    cfg = (2, 64, 512)
    res = benchmarks.bench_swiglu(configs=[cfg], warmup=2, iterations=5)
    assert list(res) == [cfg]
    r = res[cfg]
    assert set(r) == {"pytorch_ms", "hip_ms", "max_diff"}
    for key in ("pytorch_ms", "hip_ms"):
        mean, std = r[key]
        assert mean > 0 and std >= 0
    assert r["max_diff"] < 1e-2        # benchmark_swiglu.py:124-126
    out = capsys.readouterr().out
    assert "PyTorch native" in out and "Speedup" in out and "peak memory" in out


def test_swiglu_block_benchmark_default_config_list():
    from mgrrmsnorm_amd import benchmarks

    assert benchmarks.SWIGLU_CONFIGS == [(8, 128, 2048), (16, 256, 4096), (32, 512, 4096)]   # benchmark_swiglu.py:167-172
    assert benchmarks.RMSNORM_CONFIGS == [(32, 128, 4096)]


# the formula evaluated by torch in the storage type is itself off by up to an ulp of the
# output (2^-10 relative in fp16, 2^-7 in bf16; |y| reaches about 4 here)
@pytest.mark.parametrize("backward", [False, True])
@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-2), (torch.bfloat16, 6.5e-2)])
def test_rmsnorm_benchmark(dtype, tol, backward, capsys):
    from mgrrmsnorm_amd import benchmarks

    cfg = (4, 32, 1024)
    res = benchmarks.bench_rmsnorm(dtype=dtype, configs=[cfg], warmup=2, iterations=5, backward=backward)
    r = res[cfg]
    assert set(r) == {"formula_ms", "native_ms", "hip_ms", "formula_gpu_ms", "native_gpu_ms", "hip_gpu_ms", "max_diff"}
    assert all(r[k][0] > 0 for k in ("formula_ms", "native_ms", "hip_ms"))
    assert all(r[k] > 0 for k in ("formula_gpu_ms", "native_gpu_ms", "hip_gpu_ms"))
    assert r["max_diff"] < tol
    out = capsys.readouterr().out
    assert "tokens per second" in out and "GPU time (ms)" in out
    assert ("forward + backward" in out) == backward


def test_time_calls_statistics():
    from mgrrmsnorm_amd import benchmarks

    x = torch.ones(1024, device="cuda")
    mean, std = benchmarks.time_calls(lambda: x.add_(1), warmup=1, iterations=4)
    assert mean > 0 and std >= 0
    assert x[0].item() == 6     # 1 warm-up + 4 timed calls
