"""The C ABI without a GPU: the library loads, exports every function that
include/megagemm_hip.h declares, and rejects bad arguments before touching HIP (no
compute call is made here)."""
import ctypes
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "megagemm_hip.h"


@pytest.fixture(scope="module")
def lib():
    from mgrrmsnorm_amd import _lib

    if not _lib.LIB_PATH.exists():
        from mgrrmsnorm_amd import _build

        _build.build()
    return _lib.load()


TUNING_HEADER = ROOT / "include" / "megagemm_hip_tuning.h"


def _declared_in(header):
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mg_[a-z0-9_]+)\s*\(", text)))


def _declared_functions():
    return sorted(_declared_in(HEADER) + _declared_in(TUNING_HEADER))


def test_header_declares_the_expected_entry_points():
    assert _declared_in(HEADER) == sorted([
        "mg_abi_version", "mg_last_error", "mg_rmsnorm_fwd", "mg_rmsnorm_bwd_workspace", "mg_rmsnorm_bwd",
        "mg_rmsnorm_dw_reduce", "mg_rmsnorm_bwd_noalloc", "mg_swiglu_fwd", "mg_swiglu_bwd"])
    # measurement and tuning aids live in a header of their own
    assert _declared_in(TUNING_HEADER) == sorted([
        "mg_set_option", "mg_option_generation", "mg_copy_bytes", "mg_stream_probe", "mg_row_probe",
        "mg_rmsnorm_launch_info", "mg_rmsnorm_bwd_timeline"])


def test_library_exports_every_declared_symbol(lib):
    from mgrrmsnorm_amd import _lib

    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature in _lib.SIGNATURES"
    assert sorted(_lib.SIGNATURES) == _declared_functions()


def test_header_compiles_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "megagemm_hip.h"\n#include "megagemm_hip_tuning.h"\nint main(void){return MG_ABI_VERSION - 1;}\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", f"-I{HEADER.parent}", "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)
    subprocess.run(["g++", "-x", "c++", "-Wall", "-Werror", f"-I{HEADER.parent}", "-c", str(src), "-o",
                    str(tmp_path / "t2.o")], check=True)


def test_abi_version(lib):
    from mgrrmsnorm_amd import _lib

    assert lib.mg_abi_version() == _lib.ABI_VERSION == 2
    text = HEADER.read_text()
    assert re.search(r"#define\s+MG_ABI_VERSION\s+2\b", text)


def _err(lib):
    return lib.mg_last_error().decode()


FAKE = 0x1000  # a non-null, 16-byte aligned address that is never dereferenced on these paths


def test_rmsnorm_fwd_rejects_bad_arguments(lib):
    f = lib.mg_rmsnorm_fwd
    assert f(FAKE, FAKE, FAKE, FAKE, 4, 8, 1e-5, 7, None) == -1 and "dtype" in _err(lib)
    assert f(FAKE, FAKE, FAKE, FAKE, -1, 8, 1e-5, 0, None) == -1 and "rows" in _err(lib)
    assert f(FAKE, FAKE, FAKE, FAKE, 4, 0, 1e-5, 0, None) == -1 and "cols" in _err(lib)
    assert f(FAKE, FAKE, FAKE, FAKE, 4, 1 << 30, 1e-5, 0, None) == -2 and "too large" in _err(lib)
    assert f(FAKE, FAKE, FAKE, FAKE, 1 << 31, 8, 1e-5, 2, None) == -2
    assert f(None, FAKE, FAKE, FAKE, 4, 8, 1e-5, 0, None) == -1 and "NULL" in _err(lib)
    assert f(FAKE, FAKE, FAKE + 1, FAKE, 4, 8, 1e-5, 1, None) == -1 and "aligned" in _err(lib)
    # rows == 0 is valid and launches nothing (the reference fails with a launch error)
    assert f(None, None, None, None, 0, 8, 1e-5, 0, None) == 0


def test_rmsnorm_bwd_rejects_bad_arguments(lib):
    f = lib.mg_rmsnorm_bwd
    ok = dict(rows=4, cols=8, dtype=2, P=2, ld=64)
    call = lambda **kw: f(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, *(({**ok, **kw})[k] for k in ("rows", "cols", "dtype", "P", "ld")), None)
    assert call(dtype=9) == -1
    assert call(P=0) == -1 and "num_partials" in _err(lib)
    assert call(P=70000) == -1
    assert call(ld=8) == -1 and "ld" in _err(lib)
    assert call(ld=4, cols=8) == -1
    assert call(cols=100, ld=64) == -1
    assert f(FAKE, None, FAKE, FAKE, FAKE, FAKE, 4, 8, 2, 2, 64, None) == -1 and "dw_partial" in _err(lib)
    assert f(None, FAKE, FAKE, FAKE, FAKE, FAKE, 4, 8, 2, 2, 64, None) == -1 and "NULL" in _err(lib)


def test_dw_reduce_rejects_bad_arguments(lib):
    f = lib.mg_rmsnorm_dw_reduce
    assert f(None, None, 0, FAKE, 2, 64, 8, None) == -1 and "dw_f32" in _err(lib)
    assert f(FAKE, FAKE, 5, FAKE, 2, 64, 8, None) == -1 and "cast_dtype" in _err(lib)
    assert f(FAKE, None, 0, None, 2, 64, 8, None) == -1
    assert f(FAKE, None, 0, FAKE, 2, 32, 8, None) == -1
    assert f(FAKE, None, 0, FAKE, 0, 64, 8, None) == -1


def test_workspace_rejects_bad_arguments(lib):
    P, ld = ctypes.c_int64(-5), ctypes.c_int64(-5)
    f = lib.mg_rmsnorm_bwd_workspace
    assert f(4, 8, 3, ctypes.byref(P), ctypes.byref(ld)) == -1
    assert f(4, 8, 0, None, None) == -1
    assert f(0, 100, 2, ctypes.byref(P), ctypes.byref(ld)) == 0      # no device needed for rows == 0
    assert (P.value, ld.value) == (1, 128)


def test_swiglu_rejects_bad_arguments(lib):
    assert lib.mg_swiglu_fwd(FAKE, FAKE, 4, 0, 2, None) == -1 and "H" in _err(lib)
    assert lib.mg_swiglu_fwd(FAKE, FAKE, -1, 8, 2, None) == -1
    assert lib.mg_swiglu_fwd(FAKE, FAKE, 4, 8, 4, None) == -1
    assert lib.mg_swiglu_fwd(None, FAKE, 4, 8, 2, None) == -1
    assert lib.mg_swiglu_fwd(FAKE, FAKE, 4, 1 << 30, 2, None) == -2
    assert lib.mg_swiglu_fwd(FAKE, FAKE, 1 << 39, 4, 2, None) == -2
    assert lib.mg_swiglu_fwd(None, None, 0, 8, 2, None) == 0
    assert lib.mg_swiglu_bwd(FAKE, None, FAKE, 4, 8, 2, None) == -1
    assert lib.mg_swiglu_bwd(FAKE, FAKE + 2, FAKE, 4, 8, 0, None) == -1 and "aligned" in _err(lib)
    assert lib.mg_swiglu_bwd(None, None, None, 0, 8, 1, None) == 0


def test_copy_bytes_rejects_bad_arguments(lib):
    assert lib.mg_copy_bytes(FAKE, FAKE, 24, None) == -1 and "multiple of 16" in _err(lib)
    assert lib.mg_copy_bytes(FAKE, FAKE + 4, 32, None) == -1 and "aligned" in _err(lib)
    assert lib.mg_copy_bytes(None, FAKE, 32, None) == -1
    assert lib.mg_copy_bytes(None, None, 0, None) == 0
    assert lib.mg_row_probe(FAKE, FAKE, None, 4, 24, 0, None) == -1 and "multiple of 16" in _err(lib)
    assert lib.mg_row_probe(FAKE, FAKE, None, 4, 65552, 0, None) == -1
    assert lib.mg_row_probe(FAKE, FAKE, None, -1, 64, 0, None) == -1 and "rows" in _err(lib)
    assert lib.mg_row_probe(None, FAKE, None, 4, 64, 0, None) == -1
    assert lib.mg_row_probe(None, None, None, 0, 64, 0, None) == 0
    # the time-stamped backward launch: needs a records pointer and at least one row
    args = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 64, 4096, 2, 256, 4096)
    assert lib.mg_rmsnorm_bwd_timeline(*args, None, None) == -1 and "records" in _err(lib)
    assert lib.mg_rmsnorm_bwd_timeline(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 0, 4096, 2, 256, 4096, FAKE, None) == -1


def _launch_info(lib, backward, cols, dtype):
    out = [ctypes.c_int(-1) for _ in range(4)]
    assert lib.mg_rmsnorm_launch_info(backward, cols, dtype, *[ctypes.byref(o) for o in out]) == 0
    return tuple(o.value for o in out)   # (generic, threads per row, vectors per thread, workgroup threads)


@pytest.mark.parametrize("cols,dtype,fwd,bwd", [
    # 2-byte types: 8 elements per 16-byte vector
    (4096, 2, (0, 256, 2, 256), (0, 512, 1, 512)),      # metric shape: one row per 256-thread workgroup; backward one vector per thread (register ring)
    (2048, 1, (0, 128, 2, 256), (0, 256, 1, 512)),
    (4100, 2, (0, 256, 3, 256), (0, 512, 2, 512)),      # 513 vectors: 3 per thread rather than 2 half-empty
    (5120, 1, (0, 512, 2, 512), (0, 512, 2, 512)),
    (8192, 2, (0, 512, 2, 512), (0, 1024, 1, 1024)),
    (16384, 2, (0, 1024, 2, 1024), (0, 1024, 2, 1024)),
    (4099, 2, (0, 256, 3, 256), (0, 512, 2, 512)),      # odd width of a 2-byte type: same kernels, one lane moves the last element
    (100000, 1, (0, 1024, 0, 1024), (0, 1024, 0, 1024)),  # wider than registers hold: 1024 threads stream the row twice
    (100001, 1, (0, 1024, 0, 1024), (0, 1024, 0, 1024)),  # ... an odd width of a 2-byte type too
    (40000, 2, (0, 1024, 5, 1024), (0, 1024, 0, 1024)),   # the backward pass holds fewer vectors than the forward pass
    # rows of up to 1 KiB whose pitch is not a multiple of 128 bytes, and any row of up to 16
    # vectors: one vector per lane, 1 ... 64 lanes per row, -G = G row groups in flight
    (64, 2, (0, 8, -4, 256), (0, 8, -2, 512)),          # 8 vectors: 8 rows per group
    (128, 2, (0, 16, -4, 256), (0, 16, -2, 512)),       # head dimension 128
    (80, 2, (0, 16, -4, 256), (0, 16, -2, 512)),        # head dimension 80: 10 of 16 lanes
    (8, 2, (0, 1, -4, 256), (0, 1, -2, 512)),           # a single vector per row: a lane per row
    (24, 1, (0, 4, -4, 256), (0, 4, -2, 512)),          # 3 vectors on 4 lanes
    (264, 2, (0, 64, -4, 256), (0, 64, -2, 512)),       # 33 vectors, pitch 528 bytes
    (100, 2, (0, 16, -2, 256), (0, 16, -4, 512)),       # pitch 200 bytes: the last vector of a row is trimmed
    (64, 0, (0, 16, -4, 256), (0, 16, -2, 512)),
    # pitches that are multiples of 128 bytes, 17 vectors and up: several vectors per lane,
    # 8, 16 or 32 lanes per row; forward up to 4 vectors per lane (128 vectors), backward up to 2 (56)
    (256, 1, (0, 8, 4, 256), (0, 16, 2, 512)),
    (512, 2, (0, 16, 4, 256), (0, 64, 1, 512)),         # 64 vectors: backward takes one wave per row
    (768, 2, (0, 32, 3, 256), (0, 128, 1, 512)),         # 96 vectors fill three quarters of 128 lanes
    (1024, 1, (0, 32, 4, 256), (0, 128, 1, 512)),
    (1032, 2, (0, 64, 3, 256), (0, 128, 2, 512)),        # 129 vectors: one wave per row
    (1000, 2, (0, 64, 2, 256), (0, 128, 1, 512)),        # 125 vectors, pitch 2000 bytes: contiguous pieces per instruction
    # ragged rows that leave too many lanes idle, or are long, keep several vectors per lane
    (129, 1, (0, 8, 3, 256), (0, 8, 3, 512)),           # 17 vectors would idle 15 of 32 lanes
    (299, 1, (0, 16, 3, 256), (0, 16, 3, 512)),         # 598 bytes, rows only 2-byte aligned
    (999, 1, (0, 64, 2, 256), (0, 64, 2, 512)),         # 1998 bytes
    # fp32: 4 elements per vector, any width is 4-byte aligned
    (4096, 0, (0, 512, 2, 512), (0, 1024, 1, 1024)),
    (8192, 0, (0, 1024, 2, 1024), (0, 1024, 2, 1024)),  # 2048 vectors: two per thread, still a register ring
    (12288, 2, (0, 512, 3, 512), (0, 1024, 2, 1024)),
    (33, 0, (0, 8, 2, 256), (0, 8, 2, 512)),            # 132 bytes: 9 vectors would idle 7 of 16 lanes
    (16384, 0, (0, 1024, 4, 1024), (0, 1024, 4, 1024)),   # backward: the dW sums in LDS
])
def test_launch_shapes(lib, cols, dtype, fwd, bwd):
    assert _launch_info(lib, 0, cols, dtype) == fwd
    assert _launch_info(lib, 1, cols, dtype) == bwd


def test_ring_option_switches_the_backward_layout(lib):
    """"bwd_ring" = 0 gives back two vectors per thread at half the threads; -1 is automatic."""
    try:
        assert lib.mg_set_option(b"bwd_ring", 0) == 0
        assert _launch_info(lib, 1, 4096, 2) == (0, 256, 2, 512)
        assert _launch_info(lib, 1, 8192, 2) == (0, 512, 2, 512)
    finally:
        assert lib.mg_set_option(b"bwd_ring", -1) == 0
    assert _launch_info(lib, 1, 4096, 2) == (0, 512, 1, 512)
    # rows whose pitch is not a multiple of 16 bytes never take the ring
    assert _launch_info(lib, 1, 4100, 2) == (0, 512, 2, 512)
    # one 256-thread row slot per workgroup exists on request only
    try:
        assert lib.mg_set_option(b"bwd_block", 256) == 0
        assert _launch_info(lib, 1, 4096, 2) == (0, 256, 2, 256)
        assert _launch_info(lib, 1, 8192, 2) == (0, 1024, 1, 1024) or _launch_info(lib, 1, 8192, 2)[3] != 256
    finally:
        assert lib.mg_set_option(b"bwd_block", 0) == 0


def test_forward_rows_on_the_lines_of_the_output(lib):
    """"fwd_lines" = 1: pitches that are multiples of 8 but not of 128 bytes, beyond 4 KiB, take a
    shape that holds the row plus up to 120 bytes of slots in front of it; by default nothing does."""
    shapes = {          # (cols, dtype) -> (threads per row, vectors per thread)
        (4100, 2): (256, 3),     # 8200 bytes: 521 slots
        (5000, 1): (512, 2),     # 10000 bytes: 633 slots
        (2052, 2): (128, 3),     # 4104 bytes: 265 slots, the second vector of 256 threads would be empty
        (8200, 2): (512, 3),     # 16400 bytes: 1033 slots
        (12292, 1): (1024, 2),   # 24584 bytes: 1545 slots
        (2050, 0): (256, 3),     # fp32 at the pitch of 4100 two-byte columns
        (16380, 2): (1024, 3),   # 32760 bytes: 2056 slots, eight more than two vectors of 1024 threads hold
    }
    others = (4096, 4098, 4102, 2048, 1032, 2040)    # multiples of 128, not of 8, or at most 4 KiB
    default = {key: _launch_info(lib, 0, key[0], key[1]) for key in list(shapes) + [(c, 2) for c in others]}
    assert default[(16380, 2)][:3] == (0, 1024, 2)
    try:
        assert lib.mg_set_option(b"fwd_lines", 1) == 0
        for (cols, dtype), (tpr, items) in shapes.items():
            assert _launch_info(lib, 0, cols, dtype)[:3] == (0, tpr, items), (cols, dtype)
        for c in others:
            assert _launch_info(lib, 0, c, 2) == default[(c, 2)], c
        assert lib.mg_set_option(b"fwd_tpr", 512) == 0       # a forced shape switches the layout off as well
        assert _launch_info(lib, 0, 4100, 2)[:3] == (0, 512, 2)
    finally:
        assert lib.mg_set_option(b"fwd_tpr", 0) == 0
        assert lib.mg_set_option(b"fwd_lines", 0) == 0
    for key, shape in default.items():
        assert _launch_info(lib, 0, key[0], key[1]) == shape, key


def test_launch_info_rejects_bad_arguments(lib):
    out = [ctypes.c_int() for _ in range(4)]
    refs = [ctypes.byref(o) for o in out]
    assert lib.mg_rmsnorm_launch_info(0, 0, 2, *refs) == -1
    assert lib.mg_rmsnorm_launch_info(0, 128, 9, *refs) == -1
    assert lib.mg_rmsnorm_launch_info(0, 128, 2, None, None, None, None) == -1


def test_set_option(lib):
    assert lib.mg_set_option(b"no_such_key", 1) == -1 and "unknown key" in _err(lib)
    assert lib.mg_set_option(None, 1) == -1
    for key in (b"fwd_tpr", b"fwd_items", b"bwd_tpr", b"bwd_block", b"bwd_wg_per_cu", b"swiglu_unroll",
                b"force_generic", b"bwd_partials", b"bwd_partial_policy", b"fwd_lines"):
        assert lib.mg_set_option(key, 0) == 0
    for key in (b"bwd_ring", b"bwd_lds", b"bwd_prefetch", b"narrow_groups", b"xcd_group"):
        assert lib.mg_set_option(key, -1) == 0


def test_option_generation_counts_successful_changes_only(lib):
    g0 = lib.mg_option_generation()
    assert lib.mg_set_option(b"no_such_key", 1) == -1
    assert lib.mg_option_generation() == g0
    assert lib.mg_set_option(b"bwd_tpr", 0) == 0
    assert lib.mg_set_option(b"swiglu_max_units", 0) == 0
    assert lib.mg_option_generation() == g0 + 2


def test_remembered_workspace_shapes_follow_a_direct_option_change():
    """The ctypes binding remembers (partial rows, pitch) per shape; an option set by anyone,
    also not through the package, must make it ask the library again."""
    import ctypes
    import types

    from mgrrmsnorm_amd import ops_ctypes

    state = {"generation": 7, "partials": 256, "queries": 0}

    def workspace(rows, cols, code, n_part, ld):
        state["queries"] += 1
        ctypes.cast(n_part, ctypes.POINTER(ctypes.c_int64))[0] = state["partials"]
        ctypes.cast(ld, ctypes.POINTER(ctypes.c_int64))[0] = cols
        return 0

    fake = types.SimpleNamespace(mg_option_generation=lambda: state["generation"], mg_rmsnorm_bwd_workspace=workspace)
    dev = types.SimpleNamespace(index=0)
    saved = (dict(ops_ctypes._workspace_shapes), ops_ctypes._workspace_generation)
    try:
        assert ops_ctypes._bwd_workspace(fake, dev, 64, 4096, 2) == (256, 4096)
        assert ops_ctypes._bwd_workspace(fake, dev, 64, 4096, 2) == (256, 4096)
        assert state["queries"] == 1
        state["generation"], state["partials"] = 8, 512      # someone called mg_set_option
        assert ops_ctypes._bwd_workspace(fake, dev, 64, 4096, 2) == (512, 4096)
        assert state["queries"] == 2
    finally:
        ops_ctypes._workspace_shapes.clear()
        ops_ctypes._workspace_shapes.update(saved[0])
        ops_ctypes._workspace_generation = saved[1]


def test_fastdiv_matches_integer_division(tmp_path):
    """The multiply-high division the SwiGLU kernels index with, compiled for the host and
    compared with `/` over edge-case divisors and dividends."""
    src = tmp_path / "fd.cpp"
    src.write_text(r'''
#include "mg_divmod.hpp"
#include <cstdio>
#include <cstdint>
int main() {
    const uint32_t ds[] = {1,2,3,5,7,8,9,10,16,33,100,255,256,257,688,1000,1376,4095,4096,4097,11008,65535,65536,
                           65537,1000003,(1u<<24)-1,1u<<24,(1u<<30)-1,1u<<30,(1u<<31)-1,1u<<31,(1u<<31)+1,0xFFFFFFFFu};
    uint64_t x = 88172645463325252ull; long bad = 0, n = 0;
    for (uint32_t d : ds) {
        mg::FastDiv f = mg::make_fastdiv(d);
        const uint32_t fixed[] = {0,1,d-1,d,d+1,2*d-1,2*d,0x7FFFFFFFu,0x80000000u,0xFFFFFFFEu,0xFFFFFFFFu};
        for (uint32_t v : fixed) { ++n; if (mg::fastdiv(v, f) != v / d) ++bad; }
        for (int i = 0; i < 200000; ++i) {
            x ^= x << 13; x ^= x >> 7; x ^= x << 17;
            uint32_t v = (uint32_t)x; ++n;
            if (mg::fastdiv(v, f) != v / d) ++bad;
        }
    }
    std::printf("%ld %ld\n", n, bad);
    return bad != 0;
}
''')
    exe = tmp_path / "fd"
    subprocess.run(["g++", "-O2", "-std=c++17", f"-I{ROOT / 'mgrrmsnorm_amd' / 'csrc'}", str(src), "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout
