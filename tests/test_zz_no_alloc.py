"""mg_rmsnorm_bwd_noalloc (dW partials in the library's own device array, no allocation)
against mg_rmsnorm_bwd + mg_rmsnorm_dw_reduce with a caller workspace: bit-identical dx and
dW, on calls in a row that share the array, each smaller than the one before."""
import pytest
import torch

import gpu_util as U

pytestmark = pytest.mark.gpu

SCRATCH_FLOATS = (16 << 20) // 4   # MG_NOALLOC_SCRATCH_BYTES / 4
MAX_COLS = 65536                   # MG_NOALLOC_MAX_COLS


def _noalloc(dy, x, w, s, dtype, want_f32=True, want_cast=True):
    rows, cols = x.shape
    dx = torch.empty_like(x)
    dw = torch.full((cols,), float("nan"), dtype=torch.float32, device=x.device) if want_f32 else None
    dwc = torch.empty_like(w) if want_cast else None
    U.check(U.lib().mg_rmsnorm_bwd_noalloc(
        dx.data_ptr(), dw.data_ptr() if want_f32 else None, dwc.data_ptr() if want_cast else None, dy.data_ptr(),
        x.data_ptr(), w.data_ptr(), s.data_ptr(), rows, cols, U.CODES[dtype], U.stream()), "mg_rmsnorm_bwd_noalloc")
    return dx, dw, dwc


def _expected_partials(rows, cols, dtype):
    P, ld = U.bwd_workspace(rows, cols, dtype)
    return min(P, SCRATCH_FLOATS // ld)


def _same_bits(a, b):
    return torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


# each list is one sequence of calls on the shared array, the later ones smaller
SEQUENCES = [
    [(4096, 4096, "bf16"), (300, 768, "bf16")],
    [(600, 20000, "fp16"), (129, 4100, "fp16"), (7, 100, "fp16"), (3, 1, "fp16")],   # first: partial rows capped
    [(96, 16384, "fp32"), (33, 1000, "fp32")],
    [(40, 65536, "bf16"), (512, 128, "bf16")],                                       # widest accepted rows
]


@pytest.mark.parametrize("seq", SEQUENCES, ids=lambda s: "-".join(f"{r}x{c}{d}" for r, c, d in s))
def test_noalloc_matches_workspace_entry_points(seq):
    assert _expected_partials(600, 20000, "fp16") < U.bwd_workspace(600, 20000, "fp16")[0]   # the cap is exercised
    for n, (rows, cols, dtype) in enumerate(seq):
        print(f"case {rows}x{cols} {dtype}", flush=True)
        x, dy, w = (t.cuda() for t in U.rmsnorm_inputs(rows, cols, dtype, seed=7 + n))
        _, s = U.rmsnorm_fwd(x, w, 1e-6, dtype)
        P = _expected_partials(rows, cols, dtype)
        assert P >= 1
        dx_ref, dw_ref, dwc_ref, _ = U.rmsnorm_bwd(dy, x, w, s, dtype, num_partials=P)
        for _ in range(2):   # the second run finds the first run's partials in the array
            dx, dw, dwc = _noalloc(dy, x, w, s, dtype)
            torch.cuda.synchronize()
            assert _same_bits(dx, dx_ref), f"dx differs at {rows}x{cols} {dtype}"
            assert _same_bits(dw, dw_ref), f"dW (fp32) differs at {rows}x{cols} {dtype}"
            assert _same_bits(dwc, dwc_ref), f"dW (weight type) differs at {rows}x{cols} {dtype}"


def test_noalloc_either_dw_output_alone():
    rows, cols, dtype = 257, 2048, "bf16"
    x, dy, w = (t.cuda() for t in U.rmsnorm_inputs(rows, cols, dtype, seed=3))
    _, s = U.rmsnorm_fwd(x, w, 1e-6, dtype)
    dx_ref, dw_ref, dwc_ref, _ = U.rmsnorm_bwd(dy, x, w, s, dtype, num_partials=_expected_partials(rows, cols, dtype))
    dx, dw, _ = _noalloc(dy, x, w, s, dtype, want_cast=False)
    assert _same_bits(dx, dx_ref) and _same_bits(dw, dw_ref)
    dx, _, dwc = _noalloc(dy, x, w, s, dtype, want_f32=False)
    assert _same_bits(dx, dx_ref) and _same_bits(dwc, dwc_ref)


def test_noalloc_rejects_what_it_cannot_hold():
    lib = U.lib()
    t = torch.zeros(8, device="cuda")
    p = t.data_ptr()
    rc = lib.mg_rmsnorm_bwd_noalloc(p, p, None, p, p, p, p, 1, MAX_COLS + 1, 2, U.stream())
    assert rc == -2 and "maximum" in lib.mg_last_error().decode()
    rc = lib.mg_rmsnorm_bwd_noalloc(p, None, None, p, p, p, p, 1, 8, 2, U.stream())
    assert rc == -1 and "dw_f32" in lib.mg_last_error().decode()


def test_noalloc_zero_rows_gives_zero_dw():
    cols = 1000
    w = torch.ones(cols, device="cuda")
    dw = torch.full((cols,), float("nan"), device="cuda")
    U.check(U.lib().mg_rmsnorm_bwd_noalloc(None, dw.data_ptr(), None, None, None, w.data_ptr(), None, 0, cols, 0,
                                           U.stream()), "mg_rmsnorm_bwd_noalloc rows=0")
    assert (dw == 0).all()


def test_noalloc_under_graph_capture():
    """What the entry point is for: captured in a HIP graph (after one eager call, which looks
    the array's address up), every replay reproduces the eager result, with eager work, another
    shape's call on the shared array and synchronisation between the replays."""
    rows, cols, dtype = 777, 4096, "bf16"
    x, dy, w = (t.cuda() for t in U.rmsnorm_inputs(rows, cols, dtype, seed=21))
    _, s = U.rmsnorm_fwd(x, w, 1e-6, dtype)
    dx = torch.empty_like(x)
    dw = torch.empty(cols, dtype=torch.float32, device="cuda")
    dwc = torch.empty_like(w)
    L = U.lib()

    def enqueue():
        U.check(L.mg_rmsnorm_bwd_noalloc(dx.data_ptr(), dw.data_ptr(), dwc.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                         w.data_ptr(), s.data_ptr(), rows, cols, U.CODES[dtype], U.stream()),
                "mg_rmsnorm_bwd_noalloc")

    enqueue()
    torch.cuda.synchronize()
    want = (dx.clone(), dw.clone(), dwc.clone())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    x2, dy2, w2 = (t.cuda() for t in U.rmsnorm_inputs(50, 9000, "fp32", seed=22))
    _, s2 = U.rmsnorm_fwd(x2, w2, 1e-6, "fp32")
    for i in range(4):
        _noalloc(dy2, x2, w2, s2, "fp32")     # overwrites the shared array between replays
        for t in (dx, dw, dwc):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(_same_bits(a, b) for a, b in zip((dx, dw, dwc), want)), f"replay {i}"
