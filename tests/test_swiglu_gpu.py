"""SwiGLU activation parity on the GPU, through the C ABI, against the CPU oracle, the
golden vectors and, at the full benchmark size, exact properties.  Tolerances: see
tests/gpu_util.py."""
import numpy as np
import pytest
import torch

import gpu_util as U

pytestmark = pytest.mark.gpu

ALL = ["fp32", "fp16", "bf16"]


def _inputs(M, H, dtype, seed, scale=1.0):
    td = U.DTYPES[dtype]
    gu = (U.cpu_randn((M, 2 * H), seed) * scale).to(td)
    dh = U.cpu_randn((M, H), seed + 1).to(td)
    return gu, dh


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("idx", range(4))
def test_golden_vectors(golden, dtype, idx):
    c = golden["swiglu"][idx]
    td = U.DTYPES[dtype]
    gu = torch.tensor(c["gu"], dtype=torch.float64).to(td)
    dh = torch.tensor(c["dh"], dtype=torch.float64).to(td)
    assert (gu.double() == torch.tensor(c["gu"], dtype=torch.float64)).all()
    H = c["H"]
    h = U.swiglu_fwd(gu.cuda(), H, dtype)
    U.assert_matches(h, np.array(c["h"]), dtype, "h")
    d = U.swiglu_bwd(dh.cuda(), gu.cuda(), H, dtype)
    _, _, floor = U.swiglu_reference(gu, dh, dtype)
    U.assert_matches(d, np.array(c["dgu"]), dtype, "[d_gate | d_up]", floor=floor)


SHAPES = [
    (1024, 11008),   # the benchmark width at a row count the oracle handles in seconds
    (512, 6912),     # MegaGemmTriton(4096).hidden
    (300, 256),
    (33, 100),       # 200-byte half rows: not a multiple of 16 bytes for 2-byte types
    (5, 33),         # odd width: the `up` half starts misaligned
    (7, 1),
    (1, 8),
    (1, 4),
    (4097, 24),
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("M,H", SHAPES)
def test_forward_backward_match_oracle(dtype, M, H):
    gu, dh = _inputs(M, H, dtype, seed=M + H, scale=2.0)
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    gud, dhd = gu.cuda(), dh.cuda()
    U.assert_matches(U.swiglu_fwd(gud, H, dtype), h_ref, dtype, f"h {M}x{H}")
    U.assert_matches(U.swiglu_bwd(dhd, gud, H, dtype), d_ref, dtype, f"dgu {M}x{H}", floor=floor)


@pytest.mark.parametrize("dtype", ALL)
def test_extreme_gates(dtype):
    """Both tails of the sigmoid, zero, and the root of silu'."""
    gates = [0.0, -0.0, 1.0, -1.0, -1.2784645, 10.0, -10.0, 20.0, -20.0, 40.0, -40.0, 80.0, -80.0, 200.0, -200.0,
             1e-3, -1e-3, 3e4, -3e4]
    H = 24
    g = torch.tensor(gates + [0.5] * (H - len(gates)), dtype=torch.float32)
    u = torch.linspace(-2.0, 2.0, H)
    gu = torch.cat([g, u]).unsqueeze(0).repeat(3, 1).to(U.DTYPES[dtype])
    dh = torch.ones((3, H)).to(U.DTYPES[dtype])
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    h = U.swiglu_fwd(gu.cuda(), H, dtype)
    d = U.swiglu_bwd(dh.cuda(), gu.cuda(), H, dtype)
    assert torch.isfinite(h).all() and torch.isfinite(d).all()
    U.assert_matches(h, h_ref, dtype, "h")
    U.assert_matches(d, d_ref, dtype, "dgu", floor=floor)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("M,H,off", [(301, 1001, 0), (77, 1376, 3), (1000, 100, 1), (19, 7, 0), (4097, 33, 5), (9, 2049, 2)])
def test_any_width_and_alignment(dtype, M, H, off):
    """Half rows that are not whole 16-byte vectors (odd widths included) and bases `off`
    elements away from an aligned address: the 16-byte kernels for ragged rows.  Outputs sit
    between canary elements that must stay untouched."""
    td = U.DTYPES[dtype]
    gu, dh = _inputs(M, H, dtype, seed=M + 3 * H + off, scale=2.0)
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    PAD = 32

    def placed(shape, src=None):
        n = shape[0] * shape[1]
        buf = torch.full((PAD + off + n + PAD,), 7.0, dtype=td, device="cuda")
        view = buf[PAD + off: PAD + off + n].view(*shape)
        if src is not None:
            view.copy_(src)
        return buf, view, n

    _, gud, _ = placed((M, 2 * H), gu)
    _, dhd, _ = placed((M, H), dh)
    hbuf, h, hn = placed((M, H))
    dbuf, d, dn = placed((M, 2 * H))
    L = U.lib()
    U.check(L.mg_swiglu_fwd(h.data_ptr(), gud.data_ptr(), M, H, U.CODES[dtype], U.stream()))
    U.check(L.mg_swiglu_bwd(d.data_ptr(), dhd.data_ptr(), gud.data_ptr(), M, H, U.CODES[dtype], U.stream()))
    torch.cuda.synchronize()
    for buf, n in ((hbuf, hn), (dbuf, dn)):
        assert (buf[:PAD + off] == 7).all() and (buf[PAD + off + n:] == 7).all(), "wrote outside the output"
    U.assert_matches(h, h_ref, dtype, f"h {M}x{H}+{off}")
    U.assert_matches(d, d_ref, dtype, f"dgu {M}x{H}+{off}", floor=floor)


@pytest.mark.parametrize("dtype", ALL)
def test_generic_kernels_match_oracle(dtype):
    M, H = 64, 512
    gu, dh = _inputs(M, H, dtype, seed=77)
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    gud, dhd = gu.cuda(), dh.cuda()
    U.check(U.lib().mg_set_option(b"force_generic", 1))
    try:
        h = U.swiglu_fwd(gud, H, dtype)
        d = U.swiglu_bwd(dhd, gud, H, dtype)
    finally:
        U.check(U.lib().mg_set_option(b"force_generic", 0))
    U.assert_matches(h, h_ref, dtype, "h (forced generic)")
    U.assert_matches(d, d_ref, dtype, "dgu (forced generic)", floor=floor)
    # a base pointer that is not 16-byte aligned takes the any-alignment vector kernels
    pad = torch.empty(M * 2 * H + 1, dtype=U.DTYPES[dtype], device="cuda")
    gm = pad[1:].view(M, 2 * H)
    gm.copy_(gud)
    U.assert_matches(U.swiglu_fwd(gm, H, dtype), h_ref, dtype, "h (misaligned)")
    U.assert_matches(U.swiglu_bwd(dhd, gm, H, dtype), d_ref, dtype, "dgu (misaligned)", floor=floor)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8])
def test_every_unroll_factor(unroll):
    M, H = 777, 1376
    gu, dh = _inputs(M, H, "bf16", seed=5)
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, "bf16")
    U.check(U.lib().mg_set_option(b"swiglu_unroll", unroll))
    try:
        h = U.swiglu_fwd(gu.cuda(), H, "bf16")
        d = U.swiglu_bwd(dh.cuda(), gu.cuda(), H, "bf16")
    finally:
        U.check(U.lib().mg_set_option(b"swiglu_unroll", 0))
    U.assert_matches(h, h_ref, "bf16", f"h unroll={unroll}")
    U.assert_matches(d, d_ref, "bf16", f"dgu unroll={unroll}", floor=floor)


@pytest.mark.parametrize("dtype", ALL)
def test_zero_rows(dtype):
    td = U.DTYPES[dtype]
    gu = torch.empty((0, 64), dtype=td, device="cuda")
    assert U.swiglu_fwd(gu, 32, dtype).shape == (0, 32)
    assert U.swiglu_bwd(torch.empty((0, 32), dtype=td, device="cuda"), gu, 32, dtype).shape == (0, 64)
    torch.cuda.synchronize()


def test_full_size_properties():
    """Benchmark shape [8192, 2 x 11008] bf16: (a) rows are independent -- a 64-row block
    repeated gives the block's oracle-checked answer in every repetition; (b) the output is
    linear in `up` and the gradients in dh: doubling either doubles results bit-exactly."""
    M, H, blk, dtype = 8192, 11008, 64, "bf16"
    reps = M // blk
    gu, dh = _inputs(blk, H, dtype, seed=9, scale=1.5)
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    GU = gu.cuda().unsqueeze(0).expand(reps, blk, 2 * H).reshape(M, 2 * H).contiguous()
    DH = dh.cuda().unsqueeze(0).expand(reps, blk, H).reshape(M, H).contiguous()
    h = U.swiglu_fwd(GU, H, dtype)
    d = U.swiglu_bwd(DH, GU, H, dtype)
    U.assert_matches(h[:blk], h_ref, dtype, "h, first block")
    U.assert_matches(d[:blk], d_ref, dtype, "dgu, first block", floor=floor)
    assert torch.equal(h.view(reps, blk, H), h[:blk].unsqueeze(0).expand(reps, blk, H))
    assert torch.equal(d.view(reps, blk, 2 * H), d[:blk].unsqueeze(0).expand(reps, blk, 2 * H))
    GU2 = GU.clone()
    GU2[:, H:] *= 2
    assert torch.equal(U.swiglu_fwd(GU2, H, dtype), h * 2)
    d2 = U.swiglu_bwd(DH * 2, GU, H, dtype)
    assert torch.equal(d2, d * 2)


def test_graph_capture_and_replay():
    M, H, dtype = 512, 2752, "bf16"
    gu, dh = _inputs(M, H, dtype, seed=13)
    gud, dhd = gu.cuda(), dh.cuda()
    h = torch.empty((M, H), dtype=torch.bfloat16, device="cuda")
    d = torch.empty_like(gud)
    L = U.lib()

    def enqueue():
        U.check(L.mg_swiglu_fwd(h.data_ptr(), gud.data_ptr(), M, H, 2, U.stream()))
        U.check(L.mg_swiglu_bwd(d.data_ptr(), dhd.data_ptr(), gud.data_ptr(), M, H, 2, U.stream()))

    enqueue()
    torch.cuda.synchronize()
    want = (h.clone(), d.clone())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for i in range(3):
        h.zero_(); d.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(h, want[0]) and torch.equal(d, want[1]), f"replay {i}"


def test_random_shapes_match_oracle():
    rng = np.random.default_rng(5)
    for dtype in ALL:
        for _ in range(20):
            M = int(rng.integers(1, 300))
            H = int(rng.choice([rng.integers(1, 40), rng.integers(40, 3000)]))
            gu, dh = _inputs(M, H, dtype, seed=M * 31 + H, scale=2.0)
            h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
            U.assert_matches(U.swiglu_fwd(gu.cuda(), H, dtype), h_ref, dtype, f"h {M}x{H}")
            U.assert_matches(U.swiglu_bwd(dh.cuda(), gu.cuda(), H, dtype), d_ref, dtype, f"dgu {M}x{H}", floor=floor)


@pytest.mark.parametrize("limit", [1, 1000, 5000])
def test_inputs_split_over_several_launches(limit):
    """Inputs beyond 2^31 units per launch are split by rows; with the limit lowered the same
    code path runs at a size the oracle can check (vector and element-wise kernels)."""
    L = U.lib()
    for dtype, (M, H) in (("bf16", (37, 1376)), ("fp32", (53, 33)), ("fp16", (19, 100))):
        gu, dh = _inputs(M, H, dtype, seed=limit + M)
        h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
        U.check(L.mg_set_option(b"swiglu_max_units", limit))
        try:
            h = U.swiglu_fwd(gu.cuda(), H, dtype)
            d = U.swiglu_bwd(dh.cuda(), gu.cuda(), H, dtype)
        finally:
            U.check(L.mg_set_option(b"swiglu_max_units", 0))
        U.assert_matches(h, h_ref, dtype, f"h split at {limit}")
        U.assert_matches(d, d_ref, dtype, f"dgu split at {limit}", floor=floor)
