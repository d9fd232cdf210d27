"""RMSNorm parity on the GPU, through the C ABI (ctypes on raw device pointers), against
the CPU oracle on the same seeded inputs, the committed golden vectors, and -- at the full
benchmark sizes, where the oracle would take too long -- size-independent properties.
Tolerances: see tests/gpu_util.py."""
import numpy as np
import pytest
import torch

import gpu_util as U
import oracle

pytestmark = pytest.mark.gpu

ALL = ["fp32", "fp16", "bf16"]
EPS = 1e-6


def _dev(*ts):
    return [t.cuda() for t in ts]


# ------------------------------------------------------------------------ golden vectors

@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("idx", range(6))
def test_golden_vectors(golden, dtype, idx):
    c = golden["rmsnorm"][idx]
    td = U.DTYPES[dtype]
    x, dy, w = (torch.tensor(c[k], dtype=torch.float64).to(td) for k in ("x", "dy", "w"))
    assert (x.double() == torch.tensor(c["x"], dtype=torch.float64)).all()   # exact in every storage type
    xd, dyd, wd = _dev(x, dy, w)
    y, s = U.rmsnorm_fwd(xd, wd, c["eps"], dtype)
    U.assert_matches(y, np.array(c["y"]), dtype, "y")
    np.testing.assert_allclose(s.cpu().numpy(), np.array(c["inv_rms"]), rtol=1e-6)
    dx, dw, dwc, _ = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    floor = U.dx_floor(c["x"], c["dy"], c["w"], c["inv_rms"])
    U.assert_matches(dx, np.array(c["dx"]), dtype, "dx", floor=floor)
    U.assert_dw(dw, np.array(c["dw"]))


# ------------------------------------------------------------------ parity with the oracle

SHAPES = [
    (4096, 4096),    # benchmark shape (and the reference's README shape)
    (512, 8192),
    (300, 768),      # one wave per row, partly filled second vector
    (257, 2048),
    (129, 4100),     # row pitch 8200 bytes: every other row starts 8 bytes off a 16-byte boundary
    (67, 4098),      # row pitch 8196 bytes: rows are only 4-byte aligned, the last vector is ragged
    (31, 8190),
    (65, 5120),
    (33, 16384),
    (41, 10240),     # 1280 vectors of 2-byte elements: 512 threads with three vectors each
    (19, 12279),     # the same launch shape, odd width
    (7, 100),
    (5, 33),         # odd width: rows of 2-byte types end in half a dword
    (9, 4099),
    (4, 8191),
    (3, 1),
    (1, 8),
    (2, 20000),
    (3, 33000),      # wider than the register-resident kernels hold for 2-byte types
    (1000, 12),
    (2, 65536),      # the widest row the forward register-resident kernels hold for 2-byte types
    (5, 70000),      # beyond that: rows streamed twice by 1024-thread workgroups (forward and backward)
    (3, 70001),      # ... also when such a row ends in half a dword (2-byte types)
    (70, 33001),     # backward streams an odd width; 70 rows exceed the four rows a dW thread has in flight
    (300, 40002),    # backward streams (two launches: dx, dW partials), forward holds the row
    # rows narrower than a wave (pitch a multiple of 16 bytes): several rows share a wave
    (1000, 64),      # 8 lanes per row for 2-byte types; 1000 = 125 full waves of 8 rows
    (1003, 128),     # the last wave holds 3 rows of its 8
    (517, 256),      # 16 lanes per row, 2 vectors per lane
    (259, 8),        # one vector per row (2-byte types), two for fp32
    (37, 72),        # 9 vectors: the second vector of a lane exists for one lane only
    (5000, 200),     # 25 vectors over 16 lanes
    (3, 32),
    (70000, 16),     # more rows than the backward grid has row slots at once
    (4001, 100),     # pitch 200 bytes: a row's last vector reaches into the next row and is trimmed
    (3001, 127),     # odd width: rows 2-byte aligned, each ends in half a dword
    (999, 299),
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_forward_backward_match_oracle(dtype, rows, cols):
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=42 + rows + cols)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    U.assert_matches(y, y_ref, dtype, f"y {rows}x{cols}")
    np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6, err_msg="inv_rms")
    dx, dw, dwc, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    U.assert_matches(dx, dx_ref, dtype, f"dx {rows}x{cols}", floor=floor)
    U.assert_dw(dw, dw_ref)
    assert torch.isfinite(part[:, :cols]).all(), "a partial dW entry was left unwritten"
    # grad_weight as the reference returns it: the fp32 sum rounded once to the weight type
    assert torch.equal(dwc, dw.to(U.DTYPES[dtype]))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("cols", [768, 2048, 4100, 5120, 16384])
def test_outlier_rows(dtype, cols):
    """The hidden-size sweep's data: 1% of x and dy scaled by 100, at a row count the oracle
    handles in seconds."""
    rows = 1024
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=7 + cols, outliers=True)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    U.assert_matches(y, y_ref, dtype, "y")
    dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    U.assert_matches(dx, dx_ref, dtype, "dx", floor=floor)
    U.assert_dw(dw, dw_ref)


@pytest.mark.parametrize("dtype", ALL)
def test_generic_kernels_match_oracle(dtype):
    """The element-wise path forced on a shape the vector kernels would take; then the vector
    kernels on a base pointer that is aligned to the element size only."""
    rows, cols = 100, 1024
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=99)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    U.check(U.lib().mg_set_option(b"force_generic", 1))
    try:
        y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
        dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    finally:
        U.check(U.lib().mg_set_option(b"force_generic", 0))
    U.assert_matches(y, y_ref, dtype, "y (forced generic)")
    U.assert_matches(dx, dx_ref, dtype, "dx (forced generic)", floor=floor)
    U.assert_dw(dw, dw_ref)

    # misaligned: a view that starts one element into a larger buffer
    pad = torch.empty(rows * cols + 1, dtype=U.DTYPES[dtype], device="cuda")
    xm = pad[1:].view(rows, cols)
    xm.copy_(xd)
    assert xm.data_ptr() % 16 != 0
    y2, s2 = U.rmsnorm_fwd(xm, wd, EPS, dtype)
    U.assert_matches(y2, y_ref, dtype, "y (misaligned x)")
    dx2, dw2, _, _ = U.rmsnorm_bwd(dyd, xm, wd, s2, dtype)
    U.assert_matches(dx2, dx_ref, dtype, "dx (misaligned x)", floor=floor)
    U.assert_dw(dw2, dw_ref)


@pytest.mark.parametrize("dtype,rows,cols", [
    ("bf16", 37, 4100),    # pitch 8200 = 8 mod 16: every other row starts in the middle of a slot
    ("fp16", 5, 5000),     # pitch 10000 = 16 mod 128: whole slots in front of the row
    ("bf16", 33, 2052),    # 128 threads x 3 vectors
    ("bf16", 9, 8200),     # 512 threads x 3 vectors
    ("fp16", 3, 12292),    # 1024 threads x 2 vectors, pitch 24584 = 8 mod 16
    ("fp32", 7, 2050),     # fp32 at the same pitch as 4100 two-byte columns
    ("fp32", 4, 1030),     # the shortest rows that take the layout (4120 bytes)
    ("bf16", 1, 4100),
])
@pytest.mark.parametrize("y_off,x_off", [(0, 0), (8, 8), (40, 0), (120, 16), (16, "element"), (4, 0), ("element", 8)])
def test_forward_with_the_vectors_on_the_lines_of_the_output(dtype, rows, cols, y_off, x_off):
    """On request ("fwd_lines" = 1) rows whose pitch is a multiple of 8 but not of 128 bytes put
    their 16-byte vectors on the 128-byte lines of y.  y and x start `y_off` / `x_off` bytes into 128-byte aligned buffers:
    every skew of the first row, an x that is skewed differently from y, and outputs at 4 or 2
    bytes off a multiple of 8, which must fall back to vectors counted from the row's first byte.
    Bytes around y must stay untouched."""
    es = torch.empty(0, dtype=U.DTYPES[dtype]).element_size()
    y_off, x_off = (es if o == "element" else o for o in (y_off, x_off))
    x, _, w = U.rmsnorm_inputs(rows, cols, dtype, seed=cols + y_off)
    y_ref, s_ref, _, _, _ = U.rmsnorm_reference(x, x, w, EPS, dtype)
    xd, wd = _dev(x, w)
    n, guard = rows * cols, 256 // es
    td = U.DTYPES[dtype]
    xbuf = torch.zeros(n + 2 * guard, dtype=td, device="cuda")
    ybuf = torch.full((n + 2 * guard,), 7.0, dtype=td, device="cuda")
    assert xbuf.data_ptr() % 128 == 0 and ybuf.data_ptr() % 128 == 0
    xm = xbuf[guard + x_off // es: guard + x_off // es + n].view(rows, cols)
    ym = ybuf[guard + y_off // es: guard + y_off // es + n].view(rows, cols)
    xm.copy_(xd)
    s = torch.empty(rows, dtype=torch.float32, device="cuda")
    U.check(U.lib().mg_set_option(b"fwd_lines", 1))
    try:
        U.check(U.lib().mg_rmsnorm_fwd(ym.data_ptr(), s.data_ptr(), xm.data_ptr(), wd.data_ptr(), rows, cols, EPS,
                                       U.CODES[dtype], U.stream()), "mg_rmsnorm_fwd")
        torch.cuda.synchronize()
    finally:
        U.check(U.lib().mg_set_option(b"fwd_lines", 0))
    U.assert_matches(ym, y_ref, dtype, f"y (lines, y+{y_off}, x+{x_off})")
    np.testing.assert_allclose(U.as_f32(s), s_ref, rtol=2e-6)
    lo, hi = guard + y_off // es, guard + y_off // es + n
    assert bool((ybuf[:lo] == 7.0).all()) and bool((ybuf[hi:] == 7.0).all()), "a store went outside y"
    # the default layout on the same rows, to the same tolerance
    y0, _ = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    U.assert_matches(y0, y_ref, dtype, "y (default layout)")


def test_inv_rms_pointer_may_be_null():
    x, _, w = U.rmsnorm_inputs(64, 512, "bf16")
    xd, wd = _dev(x, w)
    y1, _ = U.rmsnorm_fwd(xd, wd, EPS, "bf16", want_inv_rms=True)
    y2, s2 = U.rmsnorm_fwd(xd, wd, EPS, "bf16", want_inv_rms=False)
    assert s2 is None and torch.equal(y1, y2)


@pytest.mark.parametrize("dtype", ALL)
def test_zero_rows(dtype):
    td = U.DTYPES[dtype]
    x = torch.empty((0, 256), dtype=td, device="cuda")
    w = torch.ones(256, dtype=td, device="cuda")
    y, s = U.rmsnorm_fwd(x, w, EPS, dtype)
    assert y.shape == (0, 256) and s.shape == (0,)
    dx, dw, dwc, _ = U.rmsnorm_bwd(x, x, w, s, dtype)
    torch.cuda.synchronize()
    assert dx.shape == (0, 256) and (dw == 0).all() and (dwc == 0).all()


def test_zero_input_rows_give_zero_output_and_scaled_gradient():
    rows, cols, eps = 8, 1024, 1e-4
    x = torch.zeros((rows, cols), dtype=torch.float32, device="cuda")
    dy = U.cpu_randn((rows, cols), 5).cuda()
    w = U.cpu_randn((cols,), 6).cuda()
    y, s = U.rmsnorm_fwd(x, w, eps, "fp32")
    assert (y == 0).all()
    np.testing.assert_allclose(s.cpu().numpy(), 100.0, rtol=1e-6)
    dx, dw, _, _ = U.rmsnorm_bwd(dy, x, w, s, "fp32")
    np.testing.assert_allclose(dx.cpu().numpy(), (100.0 * dy * w).cpu().numpy(), rtol=2e-6)
    assert (dw == 0).all()


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("cols", [128, 4096])
def test_non_finite_rows_behave_like_the_formula(dtype, cols):
    """A NaN makes its own row NaN; an infinity (or squares that overflow fp32) drives the
    row's scale to rsqrt(inf) = 0, so finite elements give 0 and the infinity itself NaN --
    exactly what x * rsqrt(mean(x^2) + eps) * w gives (test_rmsnorm.py:55-56 in the
    reference).  Rows that share a wave or a workgroup with such a row are untouched."""
    rows = 64
    x, _, w = U.rmsnorm_inputs(rows, cols, dtype, seed=77)
    x[3, 5] = float("nan")
    x[10, 7] = float("inf")
    x[11, 0] = float("-inf")
    if dtype != "fp16":
        x[20, 9] = 3.0e38          # finite, but its square overflows fp32
    xd, wd = _dev(x, w)
    y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    xf, wf = xd.float(), wd.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + EPS) * wf).to(U.DTYPES[dtype])
    assert torch.equal(torch.isnan(y), torch.isnan(want))
    assert torch.isnan(y[3]).all() and torch.isnan(y[10, 7]) and torch.isnan(y[11, 0])
    assert (y[10, :7] == 0).all() and (y[10, 8:] == 0).all() and float(s[10]) == 0.0
    if dtype != "fp16":
        assert (y[20] == 0).all() and float(s[20]) == 0.0
    clean = [r for r in range(rows) if r not in (3, 10, 11, 20)]
    y_ref, *_ = U.rmsnorm_reference(x[clean], None, w, EPS, dtype)
    U.assert_matches(y[clean], y_ref, dtype, "rows next to non-finite ones")


# --------------------------------------------------------------------------- determinism

@pytest.mark.parametrize("dtype,rows,cols", [("bf16", 4096, 4096), ("fp16", 2000, 5120), ("fp32", 777, 1000),
                                             ("bf16", 100003, 128), ("fp32", 50001, 64),
                                             ("bf16", 100003, 80), ("fp16", 70001, 100),    # row groups, aligned and ragged
                                             ("bf16", 3000, 16384), ("fp16", 1500, 32768), ("fp32", 1500, 12288)])  # dW sums in LDS
def test_dw_is_bit_identical_across_runs(dtype, rows, cols):
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=3)
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    first = None
    for _ in range(10):
        dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
        if first is None:
            first = (dx.clone(), dw.clone())
        else:
            assert torch.equal(first[1].view(torch.int32), dw.view(torch.int32)), "dW differs between runs"
            assert torch.equal(first[0], dx)


@pytest.mark.parametrize("rows,cols", [(515, 2048), (5003, 128)])
@pytest.mark.parametrize("P", [1, 3, 64, 1000])
def test_any_number_of_partials_gives_the_same_gradient(P, rows, cols):
    x, dy, w = U.rmsnorm_inputs(rows, cols, "bf16", seed=11)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, "bf16")
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
    dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, "bf16", num_partials=P)
    U.assert_matches(dx, dx_ref, "bf16", f"dx P={P}", floor=floor)
    U.assert_dw(dw, dw_ref)
    assert torch.isfinite(part[:, :cols]).all()


# ------------------------------------------------- full benchmark sizes: exact properties

def _tiled(block: torch.Tensor, reps: int) -> torch.Tensor:
    return block.unsqueeze(0).expand(reps, *block.shape).reshape(reps * block.shape[0], block.shape[1]).contiguous()


FULL = [
    ("bf16", 16384, 8192),    # forward+backward configuration
    # the hidden-size sweep at its full 65536 rows, both 2-byte types
    ("bf16", 65536, 768), ("fp16", 65536, 768),
    ("bf16", 65536, 2048), ("fp16", 65536, 2048),
    ("bf16", 65536, 4100), ("fp16", 65536, 4100),
    ("bf16", 65536, 5120), ("fp16", 65536, 5120),
    ("bf16", 65536, 16384), ("fp16", 65536, 16384),   # 2^31 bytes per tensor: offsets need 64 bits
    ("fp16", 8192, 32768), ("fp32", 8192, 12288),     # backward with the dW sums in LDS: 4 and 3 vectors per thread
    ("fp32", 70000, 16388),   # 4.6 GB per tensor, rows 4-byte aligned only: offsets beyond 2^32
    ("bf16", 2097152, 128),   # rows narrower than a wave, one vector per lane: 16 rows per wave in flight
    ("bf16", 2097152, 80),    # ... at a pitch of 160 bytes
    ("fp16", 1342144, 100),   # ... at a pitch of 200 bytes: every row's last vector is trimmed
    ("fp16", 1048576, 256),   # several vectors per lane: 8 rows per wave
]


@pytest.mark.parametrize("dtype,rows,cols", FULL)
def test_full_size_by_row_replication(dtype, rows, cols):
    """Rows are independent, so a matrix made of one 64-row block repeated must give that
    block's oracle-checked y and dx in every repetition (bit for bit), and reps x its dW."""
    blk = 64
    reps = rows // blk
    x, dy, w = U.rmsnorm_inputs(blk, cols, dtype, seed=1 + cols, outliers=True)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xb, dyb, wd = _dev(x, dy, w)
    X, DY = _tiled(xb, reps), _tiled(dyb, reps)
    y, s = U.rmsnorm_fwd(X, wd, EPS, dtype)
    U.assert_matches(y[:blk], y_ref, dtype, "y, first block")
    assert torch.equal(y.view(reps, blk, cols), y[:blk].unsqueeze(0).expand(reps, blk, cols)), "y differs between repetitions"
    assert torch.equal(s.view(reps, blk), s[:blk].unsqueeze(0).expand(reps, blk))
    del y
    dx, dw, _, _ = U.rmsnorm_bwd(DY, X, wd, s, dtype)
    U.assert_matches(dx[:blk], dx_ref, dtype, "dx, first block", floor=floor)
    assert torch.equal(dx.view(reps, blk, cols), dx[:blk].unsqueeze(0).expand(reps, blk, cols)), "dx differs between repetitions"
    U.assert_dw(dw, dw_ref * reps, "dW = reps x block dW")


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
def test_one_column_rows_are_all_cancellation(dtype):
    """With a single column dx = s*dy*w - x*s^3*(dy*w*x) = s*dy*w*eps/(x^2+eps): the difference of
    two terms that agree to about eps/x^2 of their size, in every element.  No fp32 evaluation of
    the reference's formula resolves that to 1 ulp of the result (its own literal restatement
    misses at most elements as well), so this shape is held to the error bound of the subtraction,
    4 * 2^-24 * (|term 1| + |term 2|), in every element, and the counts are printed: that is the
    one place where the share of elements passing through the floor is not capped."""
    rows, cols = 629, 1
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=9)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    U.assert_matches(y, y_ref, dtype, "y, one column")
    dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    n_floor = U.assert_matches(dx, dx_ref, dtype, "dx, one column", floor=floor, every_element_cancels=True)
    U.assert_dw(dw, dw_ref)
    # the same count for the reference's own arithmetic in fp32, rounded once
    ref32 = torch.from_numpy(floor.ref32.astype(np.float32)).to(U.DTYPES[dtype])
    n_ref = U.assert_matches(ref32, dx_ref, dtype, "dx, one column, reference fp32 arithmetic", floor=floor.bound,
                             every_element_cancels=True)
    print(f"one column [{dtype}]: {n_floor} of {rows} elements of dx beyond 1 ulp / 1e-5 (within the floor); "
          f"the reference's fp32 arithmetic: {n_ref}")
    assert n_floor > 0 and n_ref > 0, "this shape is expected to need the floor on both sides"


@pytest.mark.parametrize("rows,cols,outliers", [(4096, 4096, False), (1024, 8192, False), (2048, 768, True),
                                                (2048, 2048, True), (1024, 4100, True), (1024, 5120, True),
                                                (512, 16384, True)])
def test_fp32_dx_beyond_1e5_before_the_floor_at_benchmark_widths(rows, cols, outliers):
    """The benchmark configurations' widths and input recipes in fp32: how many elements of dx
    miss the 1e-5 relative bar before the cancellation floor is applied, next to the count for
    the literal fp32 restatement of the reference's arithmetic.  The kernel may need the floor at
    no more elements than 5e-3 of the tensor plus that count."""
    x, dy, w = U.rmsnorm_inputs(rows, cols, "fp32", seed=42, outliers=outliers)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, "fp32")
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, "fp32")
    dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, "fp32")
    n_floor = U.assert_matches(dx, dx_ref, "fp32", f"dx, {rows}x{cols} fp32", floor=floor)
    U.assert_dw(dw, dw_ref)
    rel = np.abs(floor.ref32.astype(np.float64) - dx_ref) > 1e-5 * np.abs(dx_ref) + 1e-37
    print(f"{rows}x{cols} fp32{' with outliers' if outliers else ''}: {n_floor} of {rows * cols} elements of dx "
          f"({n_floor / (rows * cols):.2e}) beyond 1e-5 relative before the floor; the reference's fp32 arithmetic: "
          f"{int(rel.sum())} ({rel.mean():.2e})")


@pytest.mark.parametrize("dtype,rows,cols", [("bf16", 4096, 4096), ("bf16", 16384, 8192), ("bf16", 65536, 768),
                                             ("fp32", 4096, 4096), ("bf16", 1048576, 64)])
def test_power_of_two_scaling_is_exact(dtype, rows, cols):
    """Scaling dy (or w in the forward pass) by 2 scales every product and sum by exactly 2
    in binary floating point, so outputs must scale bit-exactly: a linearity check that
    needs no oracle and runs at full size.  (Not run for fp16, whose subnormal range --
    reached by a few outputs near zero -- does not round the same way after doubling.)"""
    td = U.DTYPES[dtype]
    g = torch.Generator(device="cuda").manual_seed(5)
    X = torch.randn((rows, cols), generator=g, device="cuda").to(td)
    DY = torch.randn((rows, cols), generator=g, device="cuda").to(td)
    W = (1 + 0.02 * torch.randn((cols,), generator=g, device="cuda")).to(td)
    y1, s = U.rmsnorm_fwd(X, W, EPS, dtype)
    y2, _ = U.rmsnorm_fwd(X, W * 2, EPS, dtype)
    assert torch.equal(y2, y1 * 2)
    dx1, dw1, _, _ = U.rmsnorm_bwd(DY, X, W, s, dtype)
    dx2, dw2, _, _ = U.rmsnorm_bwd(DY * 2, X, W, s, dtype)
    assert torch.equal(dx2, dx1 * 2)
    assert torch.equal(dw2, dw1 * 2)


# ------------------------------------------------------------------- streams and graphs

def test_runs_on_the_stream_it_is_given():
    rows, cols = 2048, 4096
    x, dy, w = U.rmsnorm_inputs(rows, cols, "bf16", seed=21)
    xd, dyd, wd = _dev(x, dy, w)
    y0, s0 = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
    dx0, dw0, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s0, "bf16")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        y1, s1 = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
        dx1, dw1, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s1, "bf16")
    side.synchronize()
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1) and torch.equal(dw0, dw1)


@pytest.mark.parametrize("rows,cols", [(1024, 4096), (300, 20480)])   # the second: backward with its dW sums in dynamic LDS
def test_graph_capture_and_replay(rows, cols):
    """Forward, backward and the dW reduction captured in one HIP graph; every replay, with
    eager work and synchronisation in between, must reproduce the eager result."""
    dtype, code = "bf16", 2
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=31)
    xd, dyd, wd = _dev(x, dy, w)
    P, ld = U.bwd_workspace(rows, cols, dtype)
    y = torch.empty_like(xd); s = torch.empty(rows, device="cuda"); dx = torch.empty_like(xd)
    part = torch.empty((P, ld), device="cuda"); dw = torch.empty(cols, device="cuda")
    L = U.lib()

    def enqueue():
        st = U.stream()
        U.check(L.mg_rmsnorm_fwd(y.data_ptr(), s.data_ptr(), xd.data_ptr(), wd.data_ptr(), rows, cols, EPS, code, st))
        U.check(L.mg_rmsnorm_bwd(dx.data_ptr(), part.data_ptr(), dyd.data_ptr(), xd.data_ptr(), wd.data_ptr(),
                                 s.data_ptr(), rows, cols, code, P, ld, st))
        U.check(L.mg_rmsnorm_dw_reduce(dw.data_ptr(), None, 0, part.data_ptr(), P, ld, cols, st))

    enqueue()
    torch.cuda.synchronize()
    want = (y.clone(), dx.clone(), dw.clone())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for i in range(4):
        xd.mul_(1.0)                      # eager work between replays
        for t in (y, dx, dw):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[0]) and torch.equal(dx, want[1]) and torch.equal(dw, want[2]), f"replay {i}"


# ----------------------------------------------------------------- seeded random shapes

def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        rows = int(rng.integers(1, 400))
        cols = int(rng.choice([rng.integers(1, 64), rng.integers(64, 1200), rng.integers(1200, 9000)]))
        out.append((rows, cols))
    return out


@pytest.mark.parametrize("dtype", ALL)
def test_random_shapes_match_oracle(dtype):
    """36 seeded (rows, cols) pairs per type, odd and ragged widths included: every launch
    shape the host can choose, both kernel families, and rows that do not fill the grid."""
    for rows, cols in _random_shapes(36, seed={"fp32": 1, "fp16": 2, "bf16": 3}[dtype]):
        x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=rows * 7919 + cols)
        y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
        xd, dyd, wd = _dev(x, dy, w)
        y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
        U.assert_matches(y, y_ref, dtype, f"y {rows}x{cols}")
        dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
        U.assert_matches(dx, dx_ref, dtype, f"dx {rows}x{cols}", floor=floor)
        U.assert_dw(dw, dw_ref, f"dW {rows}x{cols}")
        assert torch.isfinite(part[:, :cols]).all(), f"partial dW not fully written at {rows}x{cols}"


@pytest.mark.parametrize("block,tpr", [(1024, 64), (1024, 256), (1024, 1024), (512, 64), (512, 128), (512, 512)])
def test_every_backward_workgroup_shape(block, tpr):
    """Launch shapes the automatic choice does not pick for this size still give the same answer."""
    rows, cols = 700, 1024                      # 128 vectors per row: 2 per thread at 64 threads per row
    x, dy, w = U.rmsnorm_inputs(rows, cols, "bf16", seed=17)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, "bf16")
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
    L = U.lib()
    U.check(L.mg_set_option(b"bwd_block", block)); U.check(L.mg_set_option(b"bwd_tpr", tpr))
    try:
        dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, "bf16")
    finally:
        U.check(L.mg_set_option(b"bwd_block", 0)); U.check(L.mg_set_option(b"bwd_tpr", 0))
    U.assert_matches(dx, dx_ref, "bf16", f"dx block={block} tpr={tpr}", floor=floor)
    U.assert_dw(dw, dw_ref)


@pytest.mark.parametrize("dtype,rows,cols", [("bf16", 1000, 4096), ("fp16", 333, 2048), ("bf16", 77, 1000), ("fp32", 500, 2048)])
def test_one_row_slot_per_workgroup_on_request(dtype, rows, cols):
    """"bwd_block" = 256: 256-thread workgroups of one row slot each, two per compute unit (an
    experiment kept reachable through the option; it measures slower than two slots sharing a
    workgroup).  Same answers; twice the partial rows."""
    import ctypes

    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=71)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    L = U.lib()
    P0, _ = U.bwd_workspace(rows, cols, dtype)
    U.check(L.mg_set_option(b"bwd_block", 256))
    try:
        out = [ctypes.c_int(0) for _ in range(4)]
        U.check(L.mg_rmsnorm_launch_info(1, cols, U.CODES[dtype], *[ctypes.byref(o) for o in out]))
        assert (out[1].value, out[3].value) == (256, 256) and out[2].value in (1, 2)
        P1, _ = U.bwd_workspace(rows, cols, dtype)
        dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    finally:
        U.check(L.mg_set_option(b"bwd_block", 0))
    assert P1 == min(2 * torch.cuda.get_device_properties(0).multi_processor_count, rows) and P1 >= P0
    U.assert_matches(dx, dx_ref, dtype, "dx bwd_block=256", floor=floor)
    U.assert_dw(dw, dw_ref)
    assert torch.isfinite(part).all()


@pytest.mark.parametrize("dtype,rows,cols", [("bf16", 4096, 4096), ("fp16", 300, 3584), ("fp32", 700, 2048)])
def test_partial_row_store_policies_agree(dtype, rows, cols):
    """"bwd_partial_policy": default, non-temporal and written-through stores of the partial rows
    (register-ring kernel on 512 threads) are the same numbers, bit for bit."""
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=72)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    L = U.lib()
    got = []
    for pol in (0, 1, 2):
        U.check(L.mg_set_option(b"bwd_partial_policy", pol))
        try:
            dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
        finally:
            U.check(L.mg_set_option(b"bwd_partial_policy", 0))
        assert torch.isfinite(part).all(), f"policy {pol}: padding columns of a partial row were left unwritten"
        got.append((dx.clone(), part.clone(), dw.clone()))
    U.assert_matches(got[0][0], dx_ref, dtype, "dx, partial policies", floor=floor)
    U.assert_dw(got[0][2], dw_ref)
    for pol in (1, 2):
        for a, b in zip(got[0], got[pol]):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"policy {pol} differs"


@pytest.mark.parametrize("prefetch", [0, 1])
@pytest.mark.parametrize("cols", [1024, 16384])
def test_backward_with_and_without_row_prefetch(prefetch, cols):
    rows = 300
    x, dy, w = U.rmsnorm_inputs(rows, cols, "bf16", seed=23)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, "bf16")
    xd, dyd, wd = _dev(x, dy, w)
    _, s = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
    U.check(U.lib().mg_set_option(b"bwd_prefetch", prefetch))
    try:
        dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, "bf16")
    finally:
        U.check(U.lib().mg_set_option(b"bwd_prefetch", -1))
    U.assert_matches(dx, dx_ref, "bf16", f"dx prefetch={prefetch}", floor=floor)
    U.assert_dw(dw, dw_ref)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("tpr", [8, 16, 32])
@pytest.mark.parametrize("cols", [32, 72, 128, 192, 256, 512, 1000, 100, 127, 299, 45])   # the last four: ragged pitches
def test_every_narrow_row_shape(dtype, tpr, cols):
    """8, 16 and 32 lanes per row with 1 to 4 vectors per lane, whichever the automatic choice
    takes; a shape that does not fit the request falls back to the automatic one."""
    rows = 333
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=31 + cols)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    L = U.lib()
    U.check(L.mg_set_option(b"fwd_tpr", tpr)); U.check(L.mg_set_option(b"bwd_tpr", tpr))
    try:
        y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
        dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    finally:
        U.check(L.mg_set_option(b"fwd_tpr", 0)); U.check(L.mg_set_option(b"bwd_tpr", 0))
    U.assert_matches(y, y_ref, dtype, f"y tpr={tpr}")
    np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6)
    U.assert_matches(dx, dx_ref, dtype, f"dx tpr={tpr}", floor=floor)
    U.assert_dw(dw, dw_ref)
    assert torch.isfinite(part).all(), "padding columns of a partial row were left unwritten"


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("groups", [1, 2, 4])
@pytest.mark.parametrize("cols", [8, 16, 24, 64, 72, 80, 128, 200, 264, 512, 1, 3, 7, 13, 45, 100, 127, 250, 500])   # from 1 on: ragged pitches
def test_every_row_group_shape(dtype, groups, cols):
    """Rows of at most 64 vectors with one vector per lane on 1 ... 64 lanes and 1, 2 or
    4 groups of rows per wave in flight, whatever the automatic choice takes; the row count
    leaves the last wave a partial block of rows."""
    import ctypes

    rows = 333
    esize = 4 if dtype == "fp32" else 2
    nvec = -(-cols * esize // 16)
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=77 + cols)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    L = U.lib()
    U.check(L.mg_set_option(b"narrow_groups", groups))
    try:
        for backward in (0, 1):
            out = [ctypes.c_int(0) for _ in range(4)]
            U.check(L.mg_rmsnorm_launch_info(backward, cols, U.CODES[dtype], *[ctypes.byref(o) for o in out]))
            if nvec <= 64 and (nvec > 4 or groups > 1):
                assert out[2].value == -groups and nvec <= out[1].value < max(2 * nvec, 2) and out[1].value in (1, 2, 4, 8, 16, 32, 64)
            else:
                assert out[2].value > 0      # too long for the layout, or fewer than 8 lanes per row with one group: ignored
        y, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
        dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    finally:
        U.check(L.mg_set_option(b"narrow_groups", -1))
    U.assert_matches(y, y_ref, dtype, f"y groups={groups}")
    np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6)
    U.assert_matches(dx, dx_ref, dtype, f"dx groups={groups}", floor=floor)
    U.assert_dw(dw, dw_ref)
    assert torch.isfinite(part).all(), "padding columns of a partial row were left unwritten"


def test_row_groups_can_be_switched_off():
    """narrow_groups = 0 sends every narrow row to the several-vectors-per-lane kernels."""
    import ctypes

    L = U.lib()
    U.check(L.mg_set_option(b"narrow_groups", 0))
    try:
        for cols in (64, 80, 100, 264):
            for backward in (0, 1):
                out = [ctypes.c_int(0) for _ in range(4)]
                U.check(L.mg_rmsnorm_launch_info(backward, cols, 2, *[ctypes.byref(o) for o in out]))
                assert out[2].value > 0 and out[1].value in (8, 16, 32, 64)
        x, dy, w = U.rmsnorm_inputs(200, 80, "bf16", seed=5)
        y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, "bf16")
        xd, dyd, wd = _dev(x, dy, w)
        y, s = U.rmsnorm_fwd(xd, wd, EPS, "bf16")
        dx, dw, _, _ = U.rmsnorm_bwd(dyd, xd, wd, s, "bf16")
    finally:
        U.check(L.mg_set_option(b"narrow_groups", -1))
    U.assert_matches(y, y_ref, "bf16", "y, groups off")
    U.assert_matches(dx, dx_ref, "bf16", "dx, groups off", floor=floor)
    U.assert_dw(dw, dw_ref)


@pytest.mark.parametrize("dtype,rows,cols,shape", [
    ("bf16", 300, 4096, (512, 1, 512)), ("bf16", 4096, 4096, (512, 1, 512)), ("fp16", 77, 768, (128, 1, 512)),
    ("bf16", 20000, 512, (64, 1, 512)), ("fp16", 1000, 2048, (256, 1, 512)), ("bf16", 530, 8192, (1024, 1, 1024)),
    ("bf16", 64, 12288, (1024, 2, 1024)), ("bf16", 700, 10240, (1024, 2, 1024)), ("fp32", 33, 8192, (1024, 2, 1024)),
    ("fp32", 1500, 1024, (256, 1, 512)), ("fp32", 259, 3072, (1024, 1, 1024)), ("bf16", 3, 6144, (1024, 1, 1024)),
    ("fp16", 513, 1000, (128, 1, 512))])
def test_backward_over_a_ring_of_register_buffers(dtype, rows, cols, shape):
    """Rows at 16-byte pitches that fill their lanes: one vector per thread (two on 1024 threads
    beyond 1024 vectors), rows kept in flight through 2 or 4 register buffers.  Both depths must
    agree bit for bit (same layout, same order of every sum) and meet the oracle; with the ring
    switched off the copying loop runs instead and meets the oracle as well."""
    import ctypes

    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=31 + cols)
    _, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    L = U.lib()
    out = [ctypes.c_int(0) for _ in range(4)]
    U.check(L.mg_rmsnorm_launch_info(1, cols, U.CODES[dtype], *[ctypes.byref(o) for o in out]))
    assert tuple(o.value for o in out[1:]) == shape
    _, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    got = {}
    for ring in (-1, 2, 4, 0):
        U.check(L.mg_set_option(b"bwd_ring", ring))
        try:
            dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
        finally:
            U.check(L.mg_set_option(b"bwd_ring", -1))
        U.assert_matches(dx, dx_ref, dtype, f"dx bwd_ring={ring}", floor=floor)
        U.assert_dw(dw, dw_ref)
        assert torch.isfinite(part).all(), "padding columns of a partial row were left unwritten"
        got[ring] = (dx.clone(), dw.clone())
    for ring in (2, 4):
        assert torch.equal(got[ring][0].view(torch.uint8), got[-1][0].view(torch.uint8)), f"dx differs at depth {ring}"
        assert torch.equal(got[ring][1].view(torch.uint8), got[-1][1].view(torch.uint8)), f"dW differs at depth {ring}"


@pytest.mark.parametrize("dtype,rows,cols", [(d, r, c) for d in ("bf16", "fp16") for r, c in
                                             [(33, 12296), (600, 16384), (21, 16383), (33, 16392), (300, 20480),
                                              (41, 24576), (19, 32768), (7, 32767), (5, 28001)]]
                         + [("fp32", 33, 8196), ("fp32", 300, 10240), ("fp32", 41, 12288), ("fp32", 19, 16384),
                            ("fp32", 7, 14001)])
def test_backward_with_the_dw_sums_in_lds(dtype, rows, cols):
    """Rows of 2049-4096 vectors (2-byte types: from 1537): 1024 threads, 2, 3 or 4 vectors each,
    dW sums in dynamic LDS; and the same rows with that switched off (sums in registers)."""
    import ctypes

    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=13 + cols)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
    xd, dyd, wd = _dev(x, dy, w)
    L = U.lib()
    out = [ctypes.c_int(0) for _ in range(4)]
    U.check(L.mg_rmsnorm_launch_info(1, cols, U.CODES[dtype], *[ctypes.byref(o) for o in out]))
    nvec = -(-cols * (4 if dtype == "fp32" else 2) // 16)
    assert [o.value for o in out] == [0, 1024, -(-nvec // 1024), 1024]
    _, s = U.rmsnorm_fwd(xd, wd, EPS, dtype)
    for lds in (-1, 0):
        U.check(L.mg_set_option(b"bwd_lds", lds))
        try:
            dx, dw, _, part = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
        finally:
            U.check(L.mg_set_option(b"bwd_lds", -1))
        U.assert_matches(dx, dx_ref, dtype, f"dx bwd_lds={lds}", floor=floor)
        U.assert_dw(dw, dw_ref)
        assert torch.isfinite(part).all(), "padding columns of a partial row were left unwritten"


@pytest.mark.parametrize("tpr", [64, 128, 256, 512, 1024])
def test_every_forward_workgroup_shape(tpr):
    rows, cols = 333, 4096
    x, _, w = U.rmsnorm_inputs(rows, cols, "fp16", seed=19)
    y_ref, s_ref, *_ = U.rmsnorm_reference(x, None, w, EPS, "fp16")
    xd, wd = _dev(x, w)
    U.check(U.lib().mg_set_option(b"fwd_tpr", tpr))
    try:
        y, s = U.rmsnorm_fwd(xd, wd, EPS, "fp16")
    finally:
        U.check(U.lib().mg_set_option(b"fwd_tpr", 0))
    U.assert_matches(y, y_ref, "fp16", f"y tpr={tpr}")
    np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6)
