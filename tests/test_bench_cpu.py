"""Host-side behaviour of bench.py that needs no GPU: argument handling, the workload names it
accepts, the byte counts behind every GB/s figure, and the source hash the profiles carry."""
import json
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))


def _run(*args):
    return subprocess.run([sys.executable, str(ROOT / "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU only" in r.stderr and "--gpus 1" in r.stderr
    assert r.stdout.strip() == ""          # no JSON line that could be mistaken for a measurement


def test_help_lists_the_launch_modes_and_the_stream_switch():
    r = _run("--help")
    assert r.returncode == 0
    for word in ("--launch", "second-stream", "--extra-streams", "--timeline", "--option", "--buffer-sets"):
        assert word in r.stdout


def test_configuration_list_covers_every_benchmark_configuration():
    import bench

    names = set(bench.CONFIGS) | {"rmsnorm_fwd_bwd_4096x4096_bf16"}      # the headline is the default workload
    assert "rmsnorm_fwd_4096x4096_fp16" in names                        # forward fp16, 4096 rows x 4096 columns
    assert "rmsnorm_fwd_bwd_16384x8192_bf16" in names                   # x [8, 2048, 8192]
    for cols in (768, 2048, 4100, 5120, 16384):                          # the hidden-size sweep at 65536 rows
        for dtype in ("bf16", "fp16"):
            assert f"rmsnorm_fwd_bwd_65536x{cols}_{dtype}" in names
    assert "swiglu_fwd_bwd_8192x11008_bf16" in names
    text = json.load(open(ROOT / "BASELINE.json"))["configs"]
    assert len(text) == 5     # the CPU case, fp16 forward, [8, 2048, 8192], the 65536-row sweep, SwiGLU
    for needle in ("4096", "8192", "65536", "11008"):
        assert any(needle in t for t in text)


def test_unknown_workload_names_are_refused():
    import bench

    for bad in ("rmsnorm_4096x4096_bf16", "rmsnorm_fwd_4096x4096_int8", "swiglu_fwd_8192x11008_bf16", ""):
        with pytest.raises(SystemExit):
            bench.make_workload(None, bad)


def test_algorithmic_bytes_are_reads_plus_writes_of_every_tensor():
    """The figures every GB/s is computed from: forward reads x and w and writes y; backward
    reads dy, x and w and writes dx and the fp32 dW (inv_rms, 4 bytes a row, is left out)."""
    import bench

    src = (ROOT / "bench.py").read_text()
    assert "self.fwd_bytes = 2 * rows * cols * e + cols * e" in src
    assert "self.bwd_bytes = 3 * rows * cols * e + cols * e + 4 * cols" in src
    rows = cols = 4096
    fwd = 2 * rows * cols * 2 + cols * 2
    bwd = 3 * rows * cols * 2 + cols * 2 + 4 * cols
    assert (fwd, bwd, fwd + bwd) == (67117056, 100687872, 167804928)     # the headline step's bytes
    assert bench.HBM_PEAK_GBPS == 8000.0


def test_profiles_carry_the_hash_of_the_sources_they_were_taken_with():
    import bench

    sha = bench.library_source_sha16()
    assert re.fullmatch(r"[0-9a-f]{16}", sha)
    stale = []
    for f in sorted((ROOT / "profiles").glob("*.md")):
        m = re.search(r"sha256\[:16\] = `([0-9a-f]{16})`", f.read_text())
        if m and m.group(1) != sha:
            stale.append(f.name)
    traffic = json.load(open(ROOT / "profiles" / "pmc_traffic.json"))
    if traffic.get("_library_source_sha16") != sha:
        stale.append("pmc_traffic.json")
    assert not stale, f"taken with other library sources than the tree holds: {stale}"
