#!/usr/bin/env python3
"""Benchmark of the RMSNorm / SwiGLU path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--launch graph|eager|second-stream]

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM.  The default workload is the one the headline metric is quoted on:
RMSNorm forward + backward (three launches: forward, backward pass 1, dW reduction) at
[4096 x 4096] bf16.  The last line printed on stdout is one JSON object; `value` is
algorithmic bytes per step / wall time per step over exactly K steps (the median of five
such readings; all five are in `readings_us_per_step`).

Buffers rotate over several independent sets whose total size exceeds the 256 MB
Infinity Cache, so consecutive steps do not find their inputs cached.

Everything runs on the default stream while it is the process's only stream; the HIP-graph
reading of the default `--launch best` comes last, because capturing a graph creates a stream
(see --extra-streams for what that changes).

Workloads: rmsnorm_fwd_bwd_4096x4096_bf16 (default), rmsnorm_fwd_4096x4096_fp16,
rmsnorm_fwd_bwd_16384x8192_bf16, rmsnorm_fwd_bwd_65536x{768,2048,4100,5120,16384}_{bf16,fp16},
swiglu_fwd_bwd_8192x11008_bf16.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import re
import sys
import time
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
ESIZE = {"fp32": 4, "fp16": 2, "bf16": 2}
CODE = {"fp32": 0, "fp16": 1, "bf16": 2}
TORCH = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
INFINITY_CACHE_BYTES = 256 << 20


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# ----------------------------------------------------------------------------- workloads

class RmsNormWorkload:
    """fwd (+ bwd + dW reduce) on [rows, cols]; inputs N(0,1), w = 1 + 0.02 N(0,1), eps 1e-6."""

    def __init__(self, lib, rows, cols, dtype, backward=True, seed=42, nsets=0):
        self.lib, self.rows, self.cols, self.dtype, self.backward = lib, rows, cols, dtype, backward
        e = ESIZE[dtype]
        self.fwd_bytes = 2 * rows * cols * e + cols * e
        self.bwd_bytes = 3 * rows * cols * e + cols * e + 4 * cols
        self.step_bytes = self.fwd_bytes + (self.bwd_bytes if backward else 0)
        per_set = (4 if backward else 2) * rows * cols * e
        self.nsets = nsets if nsets > 0 else max(2, -(-4 * INFINITY_CACHE_BYTES // per_set))
        td = TORCH[dtype]
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.w = (1 + 0.02 * torch.randn(cols, generator=g, device="cuda")).to(td)
        self.sets = []
        for _ in range(self.nsets):
            s = {"x": torch.randn((rows, cols), generator=g, device="cuda").to(td)}
            s["y"] = torch.empty_like(s["x"])
            s["inv_rms"] = torch.empty(rows, dtype=torch.float32, device="cuda")
            if backward:
                s["dy"] = torch.randn((rows, cols), generator=g, device="cuda").to(td)
                s["dx"] = torch.empty_like(s["x"])
            self.sets.append(s)
        if backward:
            P, ld = ctypes.c_int64(0), ctypes.c_int64(0)
            rc = lib.mg_rmsnorm_bwd_workspace(rows, cols, CODE[dtype], ctypes.byref(P), ctypes.byref(ld))
            assert rc == 0, lib.mg_last_error()
            self.P, self.ld = P.value, ld.value
            self.partial = torch.empty((self.P, self.ld), dtype=torch.float32, device="cuda")
            self.dw = torch.empty(cols, dtype=torch.float32, device="cuda")
        self.kernels = {"rmsnorm_fwd": self.fwd_bytes}
        if backward:
            self.kernels["rmsnorm_bwd"] = self.bwd_bytes
            self.extra_kernels = ["rmsnorm_dw_reduce"]   # timed and reported, bytes belong to rmsnorm_bwd
        self.dominant = "rmsnorm_bwd" if backward else "rmsnorm_fwd"
        self.name = f"rmsnorm_{'fwd_bwd' if backward else 'fwd'}_{rows}x{cols}_{dtype}"
        self.desc = {"rows": rows, "cols": cols, "eps": 1e-6, "launches_per_step": 3 if backward else 1}
        self.tensor_bytes = rows * cols * e
        self.row_bytes = cols * e

    def _chk(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.mg_last_error().decode())

    def fwd(self, i, st):
        s = self.sets[i % self.nsets]
        self._chk(self.lib.mg_rmsnorm_fwd(s["y"].data_ptr(), s["inv_rms"].data_ptr(), s["x"].data_ptr(),
                                          self.w.data_ptr(), self.rows, self.cols, 1e-6, CODE[self.dtype], st))

    def bwd_pass1(self, i, st):
        s = self.sets[i % self.nsets]
        self._chk(self.lib.mg_rmsnorm_bwd(s["dx"].data_ptr(), self.partial.data_ptr(), s["dy"].data_ptr(),
                                          s["x"].data_ptr(), self.w.data_ptr(), s["inv_rms"].data_ptr(), self.rows,
                                          self.cols, CODE[self.dtype], self.P, self.ld, st))

    def reduce(self, i, st):
        self._chk(self.lib.mg_rmsnorm_dw_reduce(self.dw.data_ptr(), None, 0, self.partial.data_ptr(), self.P,
                                                self.ld, self.cols, st))

    def bwd(self, i, st):
        """dx and dW: backward pass 1 followed by the dW reduction."""
        self.bwd_pass1(i, st)
        self.reduce(i, st)

    def step(self, i, st):
        self.fwd(i, st)
        if self.backward:
            self.bwd(i, st)

    def kernel(self, name):
        return {"rmsnorm_fwd": self.fwd, "rmsnorm_bwd": self.bwd_pass1, "rmsnorm_dw_reduce": self.reduce}[name]

    def probe(self, kind, i, st):
        """Plain streaming launches over this workload's own tensors: the ceiling."""
        s = self.sets[i % self.nsets]
        if kind == "copy":      # the forward pass's mix: one read, one write
            rc = self.lib.mg_stream_probe(s["y"].data_ptr(), s["x"].data_ptr(), None, self.tensor_bytes, st)
        elif kind == "2r1w":    # the backward pass's mix: two reads, one write
            rc = self.lib.mg_stream_probe(s["dx"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(), self.tensor_bytes, st)
        elif kind == "rows_copy":   # the same bytes, but a workgroup owns a whole row, one row each (forward)
            rc = self.lib.mg_row_probe(s["y"].data_ptr(), s["x"].data_ptr(), None, self.rows, self.row_bytes, 0, st)
        else:                   # ("rows_2r1w", G): whole rows on a persistent grid of G workgroups (backward pass 1)
            rc = self.lib.mg_row_probe(s["dx"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(), self.rows,
                                       self.row_bytes, kind[1], st)
        self._chk(rc)


class SwigluWorkload:
    """Activation fwd + bwd on gu [M, 2H] (N(0,1)) and dh [M, H]."""

    def __init__(self, lib, M, H, dtype, seed=42, nsets=0):
        self.lib, self.M, self.H, self.dtype = lib, M, H, dtype
        e = ESIZE[dtype]
        self.fwd_bytes, self.bwd_bytes = 3 * M * H * e, 5 * M * H * e
        self.step_bytes = self.fwd_bytes + self.bwd_bytes
        per_set = 6 * M * H * e
        self.nsets = nsets if nsets > 0 else max(2, -(-4 * INFINITY_CACHE_BYTES // per_set))
        td = TORCH[dtype]
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.sets = []
        for _ in range(self.nsets):
            s = {"gu": torch.randn((M, 2 * H), generator=g, device="cuda").to(td),
                 "dh": torch.randn((M, H), generator=g, device="cuda").to(td)}
            s["h"] = torch.empty_like(s["dh"])
            s["dgu"] = torch.empty_like(s["gu"])
            self.sets.append(s)
        self.kernels = {"swiglu_fwd": self.fwd_bytes, "swiglu_bwd": self.bwd_bytes}
        self.dominant = "swiglu_bwd"
        self.name = f"swiglu_fwd_bwd_{M}x{H}_{dtype}"
        self.desc = {"M": M, "H": H, "launches_per_step": 2}
        self.tensor_bytes = M * H * e

    def _chk(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.mg_last_error().decode())

    def fwd(self, i, st):
        s = self.sets[i % self.nsets]
        self._chk(self.lib.mg_swiglu_fwd(s["h"].data_ptr(), s["gu"].data_ptr(), self.M, self.H, CODE[self.dtype], st))

    def bwd(self, i, st):
        s = self.sets[i % self.nsets]
        self._chk(self.lib.mg_swiglu_bwd(s["dgu"].data_ptr(), s["dh"].data_ptr(), s["gu"].data_ptr(), self.M, self.H,
                                         CODE[self.dtype], st))

    def step(self, i, st):
        self.fwd(i, st)
        self.bwd(i, st)

    def kernel(self, name):
        return {"swiglu_fwd": self.fwd, "swiglu_bwd": self.bwd}[name]

    def probe(self, kind, i, st):
        s = self.sets[i % self.nsets]
        if kind == "copy":
            rc = self.lib.mg_stream_probe(s["h"].data_ptr(), s["dh"].data_ptr(), None, self.tensor_bytes, st)
        else:
            rc = self.lib.mg_stream_probe(s["h"].data_ptr(), s["gu"].data_ptr(), s["dh"].data_ptr(), self.tensor_bytes, st)
        self._chk(rc)


def make_workload(lib, name, nsets=0):
    m = re.fullmatch(r"rmsnorm_(fwd_bwd|fwd)_(\d+)x(\d+)_(fp32|fp16|bf16)", name)
    if m:
        return RmsNormWorkload(lib, int(m.group(2)), int(m.group(3)), m.group(4), backward=m.group(1) == "fwd_bwd",
                               nsets=nsets)
    m = re.fullmatch(r"swiglu_fwd_bwd_(\d+)x(\d+)_(fp32|fp16|bf16)", name)
    if m:
        return SwigluWorkload(lib, int(m.group(1)), int(m.group(2)), m.group(3), nsets=nsets)
    raise SystemExit(f"unknown workload '{name}'")


# -------------------------------------------------------------------------------- timing

def stream_ptr():
    return torch.cuda.current_stream().cuda_stream


def time_steps(wl, steps, warmup, launch, repeats=5):
    """Wall time of exactly `steps` steps, synchronised on both sides, measured `repeats`
    times (a timed region of 20 steps lasts under a millisecond, so a single reading moves
    by a few per cent).  Returns the sorted list of the readings in seconds."""
    for i in range(warmup):
        wl.step(i, stream_ptr())
    torch.cuda.synchronize()
    readings = []
    if launch == "graph":
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            st = stream_ptr()
            for i in range(steps):
                wl.step(warmup + i, st)
        graph.replay()            # untimed: first replay uploads the graph
        torch.cuda.synchronize()
        for _ in range(repeats):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            readings.append(time.perf_counter() - t0)
        return sorted(readings)
    st = stream_ptr()
    step = wl.step
    if launch == "second-stream":
        step = second_stream_step(wl)
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            step(warmup + i, st)
        torch.cuda.synchronize()
        readings.append(time.perf_counter() - t0)
    return sorted(readings)


def second_stream_step(wl):
    """A step whose dW reduction goes to a second stream, ordered after backward pass 1 by an
    event, so that it may overlap the next step's forward pass; the next pass 1 waits for it,
    since the partial rows are shared.  Same work and results as `wl.step`; measured on request
    only (`--launch second-stream`): the hand-over between the two queues costs more than the
    3 us of the reduction it hides."""
    if not getattr(wl, "backward", False):
        raise SystemExit("--launch second-stream needs an rmsnorm_fwd_bwd workload")
    main, side = torch.cuda.current_stream(), torch.cuda.Stream()
    after_pass1, after_reduce = torch.cuda.Event(), torch.cuda.Event()
    state = {"reduced": False}

    def step(i, st):
        wl.fwd(i, st)
        if state["reduced"]:
            main.wait_event(after_reduce)
        wl.bwd_pass1(i, st)
        after_pass1.record(main)
        side.wait_event(after_pass1)
        wl.reduce(i, side.cuda_stream)
        after_reduce.record(side)
        state["reduced"] = True

    return step


def time_kernel(wl, name, launches=200, fn=None):
    """Average duration of one launch of `name`, from HIP events around `launches`
    back-to-back launches on the launch stream (buffers rotating). Returns seconds."""
    fn = fn or wl.kernel(name)
    st = stream_ptr()
    for i in range(10):
        fn(i, st)
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(launches):
            fn(i, st)
        b.record()
        b.synchronize()
        t = a.elapsed_time(b) * 1e-3 / launches
        best = t if best is None else min(best, t)
    return best


def committed_traffic(kernel, workload):
    """HBM bytes per launch from the committed rocprofv3 counter summary (FETCH_SIZE +
    WRITE_SIZE, calibrated), and where that figure comes from.  It is a counter reading of an
    earlier profiler run of the same command, not of this run."""
    path = ROOT / "profiles" / "pmc_traffic.json"
    if not path.exists():
        return None, None
    try:
        table = json.loads(path.read_text())
        entry = table.get(f"{kernel}@{workload}", {})
        source = f"profiles/pmc_traffic.json (library source {table.get('_library_source_sha16', 'unknown')})"
        return entry.get("traffic_bytes"), source
    except (ValueError, AttributeError):
        return None, None


def library_source_sha16():
    """Hash of the kernel and launcher sources the library is built from (csrc/*.hip, *.hpp)."""
    import hashlib

    h = hashlib.sha256()
    for f in sorted((ROOT / "mgrrmsnorm_amd" / "csrc").glob("*.h*")):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    return h.hexdigest()[:16]


def ceiling(wl, launches=200):
    """What plain streaming kernels reach on this workload's own tensors, in this run."""
    t_copy = time_kernel(wl, None, launches, fn=lambda i, st: wl.probe("copy", i, st))
    t_2r1w = time_kernel(wl, None, launches, fn=lambda i, st: wl.probe("2r1w", i, st))
    n = wl.tensor_bytes
    out = {"tensor_bytes": n, "copy_us": round(t_copy * 1e6, 3), "copy_GB/s": round(2 * n / t_copy / 1e9, 1),
           "2r1w_us": round(t_2r1w * 1e6, 3), "2r1w_GB/s": round(3 * n / t_2r1w / 1e9, 1)}
    # The same bytes when a workgroup must own whole rows (it cannot store a row before it has
    # seen all of it): one row per workgroup as in the forward pass, and a persistent grid as in
    # backward pass 1 (best of 1, 2, 4 and 8 workgroups per compute unit).
    rb = getattr(wl, "row_bytes", 0)
    if rb and rb % 16 == 0 and rb <= 65536:
        t = time_kernel(wl, None, launches, fn=lambda i, st: wl.probe("rows_copy", i, st))
        out["rows_copy_us"] = round(t * 1e6, 3)
        out["rows_copy_GB/s"] = round(2 * n / t / 1e9, 1)
        if getattr(wl, "backward", False):
            best = None
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            for mult in (1, 2, 4, 8):
                G = cus * mult
                t = time_kernel(wl, None, launches, fn=lambda i, st: wl.probe(("rows_2r1w", G), i, st))
                if best is None or t < best[0]:
                    best = (t, G)
            out["rows_2r1w_persistent_us"] = round(best[0] * 1e6, 3)
            out["rows_2r1w_persistent_GB/s"] = round(3 * n / best[0] / 1e9, 1)
            out["rows_2r1w_persistent_workgroups"] = best[1]
    return out


def time_module_surface(rows, cols, dtype, iters=300, repeats=6):
    """Forward + backward through the nn.Module (megagemm.RMSNorm), eager, as a user calls it:
    host-side cost included.  Wall time per call over `iters` calls, inputs rotating; best and
    median of `repeats` runs.  torch's autograd engine hands the backward pass to a worker
    thread; when that thread sits on another core the hand-over costs about 20 us more per
    call than when both share a core, so the loop is also timed with the process pinned to
    one core (`fwd_bwd_one_core_*`), and with
    `torch.autograd.set_multithreading_enabled(False)`, which makes the engine run the backward
    pass on the calling thread (`fwd_bwd_caller_thread_*`): no hand-over at all, no pinning
    needed.  `torch_floor` is the same loop around `(x * 2).backward(dy)`: what torch itself
    costs."""
    import megagemm
    from mgrrmsnorm_amd import ops

    td = TORCH[dtype]
    e = ESIZE[dtype]
    norm = megagemm.RMSNorm(cols, 1e-6).cuda().to(td)
    nsets = max(2, -(-4 * INFINITY_CACHE_BYTES // (4 * rows * cols * e)))
    g = torch.Generator(device="cuda").manual_seed(7)
    xs = [torch.randn((rows, cols), generator=g, device="cuda").to(td).requires_grad_(True) for _ in range(nsets)]
    dys = [torch.randn((rows, cols), generator=g, device="cuda").to(td) for _ in range(nsets)]

    def call(i):
        x = xs[i % nsets]
        x.grad = None
        norm.weight.grad = None
        norm(x).backward(dys[i % nsets])

    def fwd_only(i):
        with torch.no_grad():
            norm(xs[i % nsets])

    def torch_floor(i):
        x = xs[i % nsets]
        x.grad = None
        (x * 2).backward(dys[i % nsets])

    def timed(fn):
        for i in range(20):
            fn(i)
        torch.cuda.synchronize()
        runs = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            for i in range(iters):
                fn(i)
            torch.cuda.synchronize()
            runs.append((time.perf_counter() - t0) / iters)
        return sorted(runs)

    out = {"binding": ops.backend(), "shape": f"{rows}x{cols} {dtype}"}
    step_bytes = 5 * rows * cols * e + 2 * cols * e + 4 * cols
    for key, fn, nbytes in (("fwd_bwd", call, step_bytes), ("fwd", fwd_only, 2 * rows * cols * e + cols * e),
                            ("torch_floor", torch_floor, 0)):
        runs = timed(fn)
        out[key + "_us_per_call"] = round(runs[0] * 1e6, 2)
        out[key + "_us_per_call_median"] = round(runs[len(runs) // 2] * 1e6, 2)
        if nbytes:
            out[key + "_GB/s"] = round(nbytes / runs[0] / 1e9, 1)
    if hasattr(torch.autograd, "set_multithreading_enabled"):
        with torch.autograd.set_multithreading_enabled(False):
            runs = timed(call)
        out["fwd_bwd_caller_thread_us_per_call"] = round(runs[0] * 1e6, 2)
        out["fwd_bwd_caller_thread_us_per_call_median"] = round(runs[len(runs) // 2] * 1e6, 2)
        out["fwd_bwd_caller_thread_GB/s"] = round(step_bytes / runs[0] / 1e9, 1)
    # The same loop with every thread of the process on one core: the calling thread and the
    # autograd engine's worker then hand over by a context switch instead of waking another
    # core, which is where the slower of the two regimes comes from.
    if hasattr(os, "sched_setaffinity"):
        saved = {}
        try:
            one = {sorted(os.sched_getaffinity(0))[0]}
            for tid in os.listdir("/proc/self/task"):
                saved[int(tid)] = os.sched_getaffinity(int(tid))
                os.sched_setaffinity(int(tid), one)
            runs = timed(call)
            out["fwd_bwd_one_core_us_per_call"] = round(runs[0] * 1e6, 2)
            out["fwd_bwd_one_core_us_per_call_median"] = round(runs[len(runs) // 2] * 1e6, 2)
            out["fwd_bwd_one_core_GB/s"] = round(step_bytes / runs[0] / 1e9, 1)
        except OSError:
            pass
        finally:
            for tid, mask in saved.items():
                try:
                    os.sched_setaffinity(tid, mask)
                except OSError:
                    pass
    return out


# The benchmark configurations other than the headline one, timed with a few launches each
# (per-kernel microseconds and algorithmic GB/s, and what the plain streaming probe reaches on
# the same tensors): fp16 forward at 4096 x 4096, the large bf16
# shape, the 65536-row hidden-size sweep in both 2-byte types, and the SwiGLU activation.
CONFIGS = (["rmsnorm_fwd_4096x4096_fp16", "rmsnorm_fwd_bwd_16384x8192_bf16"]
           + [f"rmsnorm_fwd_bwd_65536x{c}_{d}" for c in (768, 2048, 4100, 5120, 16384) for d in ("bf16", "fp16")]
           + ["swiglu_fwd_bwd_8192x11008_bf16"])


def time_configs(lib):
    import gc

    out = {}
    for name in CONFIGS:
        wl = None
        try:
            wl = make_workload(lib, name, nsets=0)
            big = wl.step_bytes > 1e9
            n_launch = 20 if big else 100
            rec = {}
            for kname, nbytes in wl.kernels.items():
                t = time_kernel(wl, kname, launches=n_launch)
                short = kname.split("_")[-1]
                rec[short + "_us"] = round(t * 1e6, 2)
                rec[short + "_GB/s"] = round(nbytes / t / 1e9)
            # the plain streaming probe on the same tensors: one read + one write, two reads + one write
            kinds = ["copy"] + (["2r1w"] if getattr(wl, "backward", True) else [])
            for kind in kinds:
                t = time_kernel(wl, None, launches=n_launch, fn=lambda i, st: wl.probe(kind, i, st))
                rec["probe_" + kind + "_GB/s"] = round((2 if kind == "copy" else 3) * wl.tensor_bytes / t / 1e9)
            # the same bytes moved by whole rows (a workgroup per row forward, a persistent grid of one
            # workgroup per compute unit backward): what whole-row ownership costs at this row length
            # (rows of 8 KiB and more: the probe gives every row a workgroup of its own, which shorter
            # rows do not fill -- the operators put several of those on one workgroup)
            rb = getattr(wl, "row_bytes", 0)
            if rb and rb % 16 == 0 and 8192 <= rb <= 65536:
                t = time_kernel(wl, None, launches=n_launch, fn=lambda i, st: wl.probe("rows_copy", i, st))
                rec["probe_rows_copy_GB/s"] = round(2 * wl.tensor_bytes / t / 1e9)
                if getattr(wl, "backward", False):
                    cus = torch.cuda.get_device_properties(0).multi_processor_count
                    t = time_kernel(wl, None, launches=n_launch, fn=lambda i, st: wl.probe(("rows_2r1w", cus), i, st))
                    rec["probe_rows_2r1w_GB/s"] = round(3 * wl.tensor_bytes / t / 1e9)
            out[name] = rec
            log(f"[bench] config {name}: {rec}")
        except Exception as exc:     # noqa: BLE001 -- one configuration must not cost the others
            out[name] = {"error": f"{type(exc).__name__}: {exc}"}
            log(f"[bench] config {name} failed: {out[name]['error']}")
        del wl
        gc.collect()
        torch.cuda.empty_cache()
    return out


SWEEP = [
    "rmsnorm_fwd_bwd_4096x4096_bf16", "rmsnorm_fwd_4096x4096_fp16", "rmsnorm_fwd_bwd_16384x8192_bf16",
    "rmsnorm_fwd_bwd_65536x768_bf16", "rmsnorm_fwd_bwd_65536x2048_fp16", "rmsnorm_fwd_bwd_65536x4100_bf16",
    "rmsnorm_fwd_bwd_65536x5120_fp16", "rmsnorm_fwd_bwd_65536x16384_bf16", "rmsnorm_fwd_bwd_16384x16384_fp32",
    # rows narrower than a wave (per-head QK-norm widths): several rows per wave
    "rmsnorm_fwd_bwd_2097152x64_bf16", "rmsnorm_fwd_bwd_1048576x128_bf16", "rmsnorm_fwd_bwd_524288x256_bf16",
    "rmsnorm_fwd_bwd_1048576x64_fp32",
    "rmsnorm_fwd_bwd_1342144x100_bf16",   # pitch 200 bytes: not a multiple of 16
    "swiglu_fwd_bwd_8192x11008_bf16",
]


def sweep(lib):
    """Per-kernel and per-step figures for every benchmark configuration."""
    import gc

    rows = []
    log(f"[sweep] {'workload':<36} " + " ".join(f"{k:>22}" for k in ("forward", "backward", "step")))
    for name in SWEEP:
        wl = make_workload(lib, name)
        big = wl.step_bytes > 1e9
        rec = {"workload": name}
        cells = []
        for kname, nbytes in wl.kernels.items():
            t = time_kernel(wl, kname, launches=50 if big else 200)
            rec[kname] = {"us": round(t * 1e6, 2), "GB/s": round(nbytes / t / 1e9, 1)}
            cells.append(f"{t * 1e6:9.1f} us {nbytes / t / 1e9:6.0f} GB/s")
        if len(cells) == 1:
            cells.append(" " * 22)
        steps = 20 if big else 100
        ts = time_steps(wl, steps, 5, "eager", repeats=1)[0] / steps
        rec["step"] = {"us": round(ts * 1e6, 2), "GB/s": round(wl.step_bytes / ts / 1e9, 1)}
        cells.append(f"{ts * 1e6:9.1f} us {wl.step_bytes / ts / 1e9:6.0f} GB/s")
        log(f"[sweep] {name:<36} " + " ".join(cells))
        rows.append(rec)
        del wl
        gc.collect()
        torch.cuda.empty_cache()
    return rows


# -------------------------------------------------------------------------- CPU baseline

def cpu_baseline(wl, budget_s=12.0):
    """The reference's PyTorch formulation on the host cores, fp32 (its CPU-runnable case),
    on a bounded sample of the same workload: at most 4096 rows, repeated for ~budget_s."""
    from oracle import torch_ref  # baseline leg only

    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(42)
    if isinstance(wl, RmsNormWorkload):
        rows = min(wl.rows, 4096)
        x = torch.randn((rows, wl.cols), generator=g)
        w = 1 + 0.02 * torch.randn(wl.cols, generator=g)
        dy = torch.randn((rows, wl.cols), generator=g)
        if wl.backward:
            fn = lambda: torch_ref.rmsnorm_fwd_bwd(x, w, dy, 1e-6)
            nbytes = 5 * rows * wl.cols * 4 + 2 * wl.cols * 4 + 4 * wl.cols
        else:
            fn = lambda: torch_ref.rmsnorm_formula(x, w, 1e-6)
            nbytes = 2 * rows * wl.cols * 4 + wl.cols * 4
        sample = f"{rows}x{wl.cols} fp32, torch CPU formula" + (" + autograd" if wl.backward else "")
    else:
        rows = min(wl.M, 1024)
        gu = torch.randn((rows, 2 * wl.H), generator=g)
        dh = torch.randn((rows, wl.H), generator=g)
        fn = lambda: torch_ref.swiglu_fwd_bwd(gu, dh)
        nbytes = 8 * rows * wl.H * 4
        sample = f"{rows}x{wl.H} fp32, torch CPU F.silu(gate)*up + autograd"
    for _ in range(3):
        fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 10 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{sample}; median of {len(times)} runs = {med * 1e3:.2f} ms; host has {os.cpu_count()} logical CPUs"}


# ------------------------------------------------------------------------------ timeline

def timeline(wl, lib, launches=40):
    """Where a launch of backward pass 1 spends its time, from the time stamps of
    mg_rmsnorm_bwd_timeline (10 ns clock, one record per workgroup): when workgroups start,
    when their sweeps over the row slots end, when they finish, on which die they ran.
    Averages over `launches` launches (buffers rotating), all in microseconds, plus what a
    launch would take if the last sweeps of every workgroup were handed out dynamically
    instead (a list-scheduling replay of the measured per-workgroup speeds)."""
    import heapq
    import statistics as st

    W = 32
    rec = torch.zeros((wl.P, W), dtype=torch.int64, device="cuda")
    runs = []
    for i in range(launches + 4):
        s = wl.sets[i % wl.nsets]
        rec.zero_()
        rc = lib.mg_rmsnorm_bwd_timeline(s["dx"].data_ptr(), wl.partial.data_ptr(), s["dy"].data_ptr(), s["x"].data_ptr(),
                                         wl.w.data_ptr(), s["inv_rms"].data_ptr(), wl.rows, wl.cols, CODE[wl.dtype],
                                         wl.P, wl.ld, rec.data_ptr(), stream_ptr())
        if rc != 0:
            raise RuntimeError(lib.mg_last_error().decode())
        torch.cuda.synchronize()
        if i >= 4:
            runs.append(rec.cpu().numpy().copy())
    n_it = int((runs[0][0, 1:25] > 0).sum())
    us = lambda ticks: ticks * 0.01
    out = {"workgroups": wl.P, "sweeps_per_workgroup": n_it, "launches": launches}
    first, med_end, last_end, start_spread, sweep = [], [], [], [], []
    per_wg = [[] for _ in range(wl.P)]
    what_if = {}
    for r in runs:
        t0 = r[:, 0].min()
        start, its, loop_end, end = r[:, 0] - t0, r[:, 1:1 + n_it] - t0, r[:, W - 3] - t0, r[:, W - 2] - t0
        start_spread.append(us(start.max()))
        first.append(us(float(sorted(its[:, 0])[wl.P // 2])))
        med_end.append(us(float(sorted(end)[wl.P // 2])))
        last_end.append(us(float(end.max())))
        sweep.append(us(float(((its[:, -1] - its[:, 0]) / max(n_it - 1, 1)).mean())))
        for g in range(wl.P):
            per_wg[g].append(us(float(end[g])))
        # replay: the first K sweeps as measured, the remaining (n_it - K) * P sweeps handed to whichever
        # workgroup is free first, each at that workgroup's own mean sweep time plus `flush` for the partial
        # row a dynamically assigned unit would have to write (16 KiB) -- what dynamic scheduling could gain
        for K in (n_it, n_it - 1, n_it - 2, n_it // 2):
            for flush in (0.0, 0.2, 0.4):
                per = us((its[:, -1] - start) / n_it)
                heap = [(us(float(its[g, K - 1])) if K > 0 else us(float(start[g])), g) for g in range(wl.P)]
                heapq.heapify(heap)
                fin = [h[0] for h in sorted(heap, key=lambda h: h[1])]
                for _ in range((n_it - K) * wl.P):
                    t, g = heapq.heappop(heap)
                    t += float(per[g]) + flush
                    fin[g] = t
                    heapq.heappush(heap, (t, g))
                tail = us(float((end - its[:, -1]).mean()))
                what_if.setdefault(f"static_sweeps={K},flush_us={flush}", []).append(max(fin) + tail)
    mean = lambda v: round(sum(v) / len(v), 2)
    out.update({"start_spread_us": mean(start_spread), "first_sweep_end_median_us": mean(first),
                "steady_sweep_us": mean(sweep), "median_workgroup_end_us": mean(med_end),
                "last_workgroup_end_us": mean(last_end)})
    means = [sum(v) / len(v) for v in per_wg]
    out["per_workgroup_mean_end_us"] = {"min": round(min(means), 2), "max": round(max(means), 2),
                                        "std_of_means": round(st.pstdev(means), 2),
                                        "mean_std_across_launches": round(sum(st.pstdev(v) for v in per_wg) / wl.P, 2)}
    xcc = runs[-1][:, W - 1]
    out["mean_end_us_by_die"] = {int(d): round(sum(m for m, x in zip(means, xcc) if x == d) / max(1, int((xcc == d).sum())), 2)
                                 for d in sorted(set(int(v) for v in xcc))}
    out["replay_last_end_us"] = {k: mean(v) for k, v in what_if.items()}
    return out


# ---------------------------------------------------------------------------------- main

def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="rmsnorm_fwd_bwd_4096x4096_bf16")
    ap.add_argument("--launch", choices=["graph", "eager", "best", "second-stream"], default="best",
                    help="how the K timed steps are enqueued: one HIP graph, one by one, or the faster of the two; "
                         "'second-stream' enqueues them one by one with the dW reduction on a second stream "
                         "(measured on request only: it is slower)")
    ap.add_argument("--buffer-sets", type=int, default=0,
                    help="input/output buffer sets the steps rotate over; 0 = enough to exceed four times the "
                         "256 MiB Infinity Cache (the reported configuration), 1 = everything stays cache resident")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="tuning override passed to mg_set_option before anything is timed (repeatable)")
    ap.add_argument("--surface", choices=["abi", "module"], default="abi",
                    help="'module' also times forward+backward through megagemm.RMSNorm (eager, host cost included) "
                         "at the workload's shape; the default run reports it for the headline shape anyway")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the per-kernel figures of the other benchmark configurations ('configs' in the JSON)")
    ap.add_argument("--sweep", action="store_true",
                    help="additionally time every configuration of the hidden-size sweep, the large RMSNorm shape "
                         "and the SwiGLU shape (per-kernel and per-step GB/s, table on stderr, 'sweep' in the JSON)")
    ap.add_argument("--timeline", type=int, default=0, metavar="LAUNCHES",
                    help="also run backward pass 1 that many times with per-workgroup time stamps "
                         "(mg_rmsnorm_bwd_timeline; shapes of 4096 two-byte columns) and report where a launch spends "
                         "its time ('timeline' in the JSON)")
    ap.add_argument("--extra-streams", type=int, default=0, metavar="N",
                    help="create N more HIP streams (one small launch on each) before anything is timed; the timed "
                         "launches stay on the default stream.  For seeing how the number of streams a process holds "
                         "changes launches with tens of thousands of workgroups")
    ap.add_argument("--calibrate-copies", type=int, default=0,
                    help="also launch this many plain copies of one activation tensor (mg_copy_bytes), so that a "
                         "counter profile of this run holds a kernel of known HBM traffic, and as many streaming "
                         "probes of each kind (mg_stream_probe) over the workload's tensors")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this build measures one GPU only (the path has no cross-GPU step); "
                         "run with --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")

    from mgrrmsnorm_amd import _lib
    lib = _lib.load()
    torch.cuda.set_device(0)
    for kv in args.option:
        key, _, val = kv.partition("=")
        _lib.set_option(key, int(val))
    wl = make_workload(lib, args.workload, args.buffer_sets)
    log(f"[bench] {wl.name}: {wl.step_bytes / 1e6:.1f} MB algorithmic per step, {wl.nsets} buffer sets, "
        f"device {torch.cuda.get_device_name(0)}")
    # The default stream has been used by now (the workload's tensors were filled on it), so its
    # hardware queue is the oldest one; every stream created here adds a newer queue.
    extra_streams = [torch.cuda.Stream() for _ in range(args.extra_streams)]
    for s_ in extra_streams:        # kept alive to the end: each holds a hardware queue once used
        with torch.cuda.stream(s_):
            torch.zeros(64, device="cuda")
        torch.cuda.synchronize()

    if args.calibrate_copies > 0:
        first = wl.sets[0]
        src_key, dst_key = ("x", "y") if "x" in first else ("dh", "h")
        nbytes = first[src_key].numel() * first[src_key].element_size()
        for i in range(args.calibrate_copies):
            s_ = wl.sets[i % wl.nsets]
            rc = lib.mg_copy_bytes(s_[dst_key].data_ptr(), s_[src_key].data_ptr(), nbytes, stream_ptr())
            assert rc == 0, lib.mg_last_error()
            wl.probe("copy", i, stream_ptr())      # the streaming yardsticks, so a profile holds them too
            wl.probe("2r1w", i, stream_ptr())
        torch.cuda.synchronize()
        log(f"[bench] calibration: {args.calibrate_copies} copies of {nbytes} bytes (traffic 2 x {nbytes} each)")

    # "best" measures the steps launched one by one first and as one HIP graph last, after every
    # other section: capturing a graph makes torch create a stream, and on this machine the number
    # of streams a process holds changes what launches with tens of thousands of workgroups cost on
    # the default stream (--extra-streams shows it), so everything else is measured while the
    # default stream is the only one.
    wall, readings = {}, {}

    def measure(mode):
        readings[mode] = time_steps(wl, args.steps, args.warmup, mode)
        wall[mode] = readings[mode][len(readings[mode]) // 2]      # the median reading
        log(f"[bench] {mode}: {wall[mode] / args.steps * 1e6:.2f} us/step")

    out = {}

    def headline():
        mode = min(wall, key=wall.get)
        sec_per_step = wall[mode] / args.steps
        value = wl.step_bytes / sec_per_step / 1e9
        out.update({
            "metric": "RMSNorm fwd+bwd HBM GB/s at [4096x4096] bf16" if wl.name == "rmsnorm_fwd_bwd_4096x4096_bf16"
                      else f"{wl.name} HBM GB/s",
            "value": round(value, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 6),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": wl.dtype, "data": "synthetic",
            "config": {"workload": wl.name, **wl.desc, "buffer_sets": wl.nsets, "launch": mode},
            "launch_modes_us_per_step": {m: round(t / args.steps * 1e6, 3) for m, t in wall.items()},
            "readings_us_per_step": {m: [round(t / args.steps * 1e6, 3) for t in r] for m, r in readings.items()},
            "library_source_sha16": library_source_sha16(),
        })

    measure("eager" if args.launch == "best" else args.launch)
    # The headline figures stand from here on; everything below adds detail to the same JSON line
    # (the graph reading of "best" may still replace them if it is the faster one), and a failure
    # in one of those sections is recorded under its key instead of losing the line.
    headline()

    def section(key, fn):
        try:
            out[key] = fn()
        except Exception as exc:     # noqa: BLE001 -- recorded, the line is still printed
            out[key] = {"error": f"{type(exc).__name__}: {exc}"}
            log(f"[bench] section '{key}' failed: {out[key]['error']}")
            try:
                torch.cuda.synchronize()
            except Exception:        # noqa: BLE001
                pass
        return out[key]

    def kernels_and_roofline():
        kern = {}
        for name, nbytes in wl.kernels.items():
            t = time_kernel(wl, name)
            kern[name] = {"us": round(t * 1e6, 3), "GB/s": round(nbytes / t / 1e9, 1), "bytes": nbytes}
            log(f"[bench] kernel {name}: {t * 1e6:.2f} us/launch, {nbytes / t / 1e9:.0f} GB/s")
        for name in getattr(wl, "extra_kernels", []):
            t = time_kernel(wl, name)
            kern[name] = {"us": round(t * 1e6, 3)}
            log(f"[bench] kernel {name}: {t * 1e6:.2f} us/launch")
        out["kernels"] = kern
        dom = wl.dominant
        achieved = kern[dom]["GB/s"]
        traffic, traffic_source = committed_traffic(dom, wl.name)
        return {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "algorithmic_bytes": kern[dom]["bytes"], "avg_launch_us": kern[dom]["us"]}

    try:
        section("roofline", kernels_and_roofline)
        log(f"[bench] ceiling on the same tensors: {section('ceiling', lambda: ceiling(wl))}")
        if isinstance(wl, RmsNormWorkload) and (args.surface == "module" or not args.no_configs):
            log(f"[bench] nn.Module surface: {section('module', lambda: time_module_surface(wl.rows, wl.cols, wl.dtype))}")
        if args.timeline > 0:
            log(f"[bench] timeline of backward pass 1: {section('timeline', lambda: timeline(wl, lib, args.timeline))}")
        if not args.no_cpu_baseline:
            log(f"[bench] cpu baseline: {section('cpu_baseline', lambda: cpu_baseline(wl))}")
        if not args.no_configs:
            section("configs", lambda: time_configs(lib))
        if args.sweep:
            section("sweep", lambda: sweep(lib))
        if args.launch == "best":
            try:
                measure("graph")
                headline()
            except RuntimeError as exc:      # the eager measurement stands
                log(f"[bench] graph launch not measured: {exc}")
                torch.cuda.synchronize()
    finally:
        print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
