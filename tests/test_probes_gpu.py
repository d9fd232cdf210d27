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
