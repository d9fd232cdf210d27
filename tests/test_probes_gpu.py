"""The library's streaming probes (measurement aids: what plain loads and stores reach on this
machine) move exactly the bytes they say they move: dst = a, or dst = a + b on 32-bit words."""
import pytest
import torch

import gpu_util as U

pytestmark = pytest.mark.gpu


def _ints(n, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randint(-2 ** 30, 2 ** 30, (n,), generator=g, device="cuda", dtype=torch.int32)


@pytest.mark.parametrize("nbytes", [16, 4096, 4112, 1 << 20, (1 << 20) + 48])
def test_stream_probe_copies_and_adds(nbytes):
    L = U.lib()
    n = nbytes // 4
    a, b = _ints(n, 1), _ints(n, 2)
    dst = torch.full((n + 8,), 7, device="cuda", dtype=torch.int32)
    U.check(L.mg_stream_probe(dst.data_ptr(), a.data_ptr(), None, nbytes, U.stream()))
    assert torch.equal(dst[:n], a) and (dst[n:] == 7).all()
    U.check(L.mg_stream_probe(dst.data_ptr(), a.data_ptr(), b.data_ptr(), nbytes, U.stream()))
    assert torch.equal(dst[:n], a + b) and (dst[n:] == 7).all()


@pytest.mark.parametrize("rows,row_bytes", [(1, 16), (37, 160), (333, 8192), (100, 8208), (19, 32768), (5, 65536)])
@pytest.mark.parametrize("workgroups", [0, 1, 7, 1000])
def test_row_probe_copies_and_adds(rows, row_bytes, workgroups):
    L = U.lib()
    n = rows * row_bytes // 4
    a, b = _ints(n, 3), _ints(n, 4)
    dst = torch.full((n + 8,), 7, device="cuda", dtype=torch.int32)
    print(f"row probe {rows} x {row_bytes} bytes, {workgroups} workgroups", flush=True)
    U.check(L.mg_row_probe(dst.data_ptr(), a.data_ptr(), None, rows, row_bytes, workgroups, U.stream()))
    assert torch.equal(dst[:n], a) and (dst[n:] == 7).all()
    U.check(L.mg_row_probe(dst.data_ptr(), a.data_ptr(), b.data_ptr(), rows, row_bytes, workgroups, U.stream()))
    assert torch.equal(dst[:n], a + b) and (dst[n:] == 7).all()


@pytest.mark.parametrize("dtype,rows,cols", [("bf16", 4096, 4096), ("fp16", 700, 4000), ("fp32", 300, 2048)])
def test_backward_timeline_gives_the_same_results_and_sane_time_stamps(dtype, rows, cols):
    """mg_rmsnorm_bwd_timeline is mg_rmsnorm_bwd with a clock: dx and the partial rows are
    bit-identical, every workgroup's record is ordered in time and names one of the 8 dies."""
    L = U.lib()
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=3)
    xd, dyd, wd = x.cuda(), dy.cuda(), w.cuda()
    _, s = U.rmsnorm_fwd(xd, wd, 1e-6, dtype)
    dx_ref, _, _, part_ref = U.rmsnorm_bwd(dyd, xd, wd, s, dtype)
    P, ld = U.bwd_workspace(rows, cols, dtype)
    dx = torch.empty_like(xd)
    part = torch.full((P, ld), float("nan"), dtype=torch.float32, device="cuda")
    rec = torch.zeros((P, 32), dtype=torch.int64, device="cuda")
    U.check(L.mg_rmsnorm_bwd_timeline(dx.data_ptr(), part.data_ptr(), dyd.data_ptr(), xd.data_ptr(), wd.data_ptr(),
                                      s.data_ptr(), rows, cols, U.CODES[dtype], P, ld, rec.data_ptr(), U.stream()))
    torch.cuda.synchronize()
    assert torch.equal(dx.view(torch.uint8), dx_ref.view(torch.uint8))
    assert torch.equal(part.view(torch.int32), part_ref.view(torch.int32))
    r = rec.cpu()
    sweeps = -(-rows // P)
    n = min(sweeps, 24)
    assert (r[:, 0] > 0).all() and (r[:, 31] >= 0).all() and (r[:, 31] < 8).all()
    seq = torch.cat([r[:, 0:1], r[:, 1:1 + n], r[:, 29:31]], dim=1)
    assert (seq[:, 1:] >= seq[:, :-1]).all(), "time stamps of a workgroup are not in order"
    assert (r[:, 1 + n:25] == 0).all() or sweeps % 4 != 0   # the loop runs a multiple of its depth
    span_us = (r[:, 30].max() - r[:, 0].min()).item() * 0.01
    print(f"{dtype} {rows}x{cols}: {P} workgroups, {sweeps} sweeps, first start to last end {span_us:.2f} us")
    assert 0 < span_us < 5000


def test_backward_timeline_refuses_shapes_without_a_time_stamped_build():
    L = U.lib()
    rows, cols = 64, 8192     # 1024 threads per row: no such build
    x, dy, w = U.rmsnorm_inputs(rows, cols, "bf16", seed=3)
    xd, dyd, wd = x.cuda(), dy.cuda(), w.cuda()
    _, s = U.rmsnorm_fwd(xd, wd, 1e-6, "bf16")
    P, ld = U.bwd_workspace(rows, cols, "bf16")
    dx = torch.empty_like(xd)
    part = torch.empty((P, ld), dtype=torch.float32, device="cuda")
    rec = torch.zeros((P, 32), dtype=torch.int64, device="cuda")
    rc = L.mg_rmsnorm_bwd_timeline(dx.data_ptr(), part.data_ptr(), dyd.data_ptr(), xd.data_ptr(), wd.data_ptr(),
                                   s.data_ptr(), rows, cols, U.CODES["bf16"], P, ld, rec.data_ptr(), U.stream())
    assert rc == -2 and "time-stamped build" in L.mg_last_error().decode()
    torch.cuda.synchronize()
