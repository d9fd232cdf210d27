"""A bounded, seeded sweep over many shapes per operator and type, through the C ABI, against
the oracle: widths of every class the launch rules distinguish (a few elements, per-head
widths, ragged and odd widths, thousands of columns up to 17000), base pointers 0-8 elements
off the allocation's alignment, and every output surrounded by canary elements so that a
store outside the tensor shows.  Each case is printed before it runs.

MG_PARITY_CASES (cases per type and operator, default 120) and MG_PARITY_SEED (added to the
seeds, default 0) widen or move the sweep for a one-off longer run."""
import os

import numpy as np
import pytest
import torch

import gpu_util as U

pytestmark = pytest.mark.gpu

EPS = 1e-6
PAD = 64
CASES_PER_DTYPE = int(os.environ.get("MG_PARITY_CASES", "120"))
SEED_SHIFT = int(os.environ.get("MG_PARITY_SEED", "0"))


def _padded(shape, td, off, src=None):
    """A [rows, cols] view `off` elements into a canary-filled buffer, and that buffer."""
    n = shape[0] * shape[1]
    buf = torch.full((PAD + off + n + PAD,), 7.0, dtype=td, device="cuda")
    view = buf[PAD + off: PAD + off + n].view(*shape)
    if src is not None:
        view.copy_(src)
    return buf, view, n


def _canaries_intact(buf, off, n):
    return bool((buf[:PAD + off] == 7).all() and (buf[PAD + off + n:] == 7).all())


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
def test_rmsnorm_many_shapes(dtype):
    rng = np.random.default_rng({"bf16": 101, "fp16": 202, "fp32": 303}[dtype] + SEED_SHIFT)
    td = U.DTYPES[dtype]
    L = U.lib()
    for i in range(CASES_PER_DTYPE):
        kind = int(rng.integers(0, 5))
        if kind == 0:
            cols = int(rng.integers(1, 40)) * 8           # per-head widths: several rows per wave
        elif kind == 1:
            cols = int(rng.integers(1, 130))              # anything small, odd widths included
        elif kind == 2:
            cols = int(rng.integers(130, 2100))
        elif kind == 3:
            cols = int(rng.integers(2100, 17000))
        else:
            cols = int(rng.choice([64, 128, 256, 512, 1024, 4096, 8192])) + int(rng.choice([0, 0, 2, 4, 8]))
        rows = int(rng.integers(1, 900 if cols < 600 else 120))
        off = int(rng.choice([0, 0, 1, 2, 3, 4, 8]))
        seed = int(rng.integers(1 << 30))
        print(f"rmsnorm {dtype} case {i}: {rows}x{cols} offset {off} seed {seed}", flush=True)
        x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=seed)
        y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, EPS, dtype)
        _, xd, n = _padded((rows, cols), td, off, x)
        _, dyd, _ = _padded((rows, cols), td, off, dy)
        wd = w.cuda()
        ybuf, y, _ = _padded((rows, cols), td, off)
        dxbuf, dx, _ = _padded((rows, cols), td, off)
        s = torch.empty(rows, dtype=torch.float32, device="cuda")
        U.check(L.mg_rmsnorm_fwd(y.data_ptr(), s.data_ptr(), xd.data_ptr(), wd.data_ptr(), rows, cols, EPS,
                                 U.CODES[dtype], U.stream()))
        P, ld = U.bwd_workspace(rows, cols, dtype)
        part = torch.full((P, ld), float("nan"), dtype=torch.float32, device="cuda")
        U.check(L.mg_rmsnorm_bwd(dx.data_ptr(), part.data_ptr(), dyd.data_ptr(), xd.data_ptr(), wd.data_ptr(),
                                 s.data_ptr(), rows, cols, U.CODES[dtype], P, ld, U.stream()))
        dw = torch.empty(cols, dtype=torch.float32, device="cuda")
        U.check(L.mg_rmsnorm_dw_reduce(dw.data_ptr(), None, 0, part.data_ptr(), P, ld, cols, U.stream()))
        torch.cuda.synchronize()
        where = f"{rows}x{cols} offset {off}"
        assert _canaries_intact(ybuf, off, n) and _canaries_intact(dxbuf, off, n), f"store outside the tensor at {where}"
        U.assert_matches(y.contiguous(), y_ref, dtype, "y, many shapes")
        np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6, err_msg=where)
        # one column: dx = s*dy*w*eps/(x^2+eps), the difference of two equal terms in every element
        U.assert_matches(dx.contiguous(), dx_ref, dtype, "dx, one column" if cols == 1 else "dx, many shapes",
                         floor=floor, every_element_cancels=cols == 1)
        U.assert_dw(dw, dw_ref, f"dW {where}")


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
def test_swiglu_many_shapes(dtype):
    rng = np.random.default_rng({"bf16": 404, "fp16": 505, "fp32": 606}[dtype] + SEED_SHIFT)
    td = U.DTYPES[dtype]
    L = U.lib()
    for i in range(CASES_PER_DTYPE):
        kind = int(rng.integers(0, 4))
        H = int([rng.integers(1, 40), rng.integers(1, 60) * 8, rng.integers(40, 3000),
                 rng.choice([1024, 4096, 6912, 11008])][kind])
        M = int(rng.integers(1, 400 if H < 1000 else 60))
        off = int(rng.choice([0, 0, 1, 2, 4, 8]))
        seed = int(rng.integers(1 << 30))
        print(f"swiglu {dtype} case {i}: {M}x{H} offset {off} seed {seed}", flush=True)
        g = torch.Generator().manual_seed(seed)
        gu = (2.0 * torch.randn((M, 2 * H), generator=g)).to(td)
        dh = torch.randn((M, H), generator=g).to(td)
        h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
        _, gud, _ = _padded((M, 2 * H), td, off, gu)
        _, dhd, _ = _padded((M, H), td, off, dh)
        hbuf, h, hn = _padded((M, H), td, off)
        dbuf, d, dn = _padded((M, 2 * H), td, off)
        U.check(L.mg_swiglu_fwd(h.data_ptr(), gud.data_ptr(), M, H, U.CODES[dtype], U.stream()))
        U.check(L.mg_swiglu_bwd(d.data_ptr(), dhd.data_ptr(), gud.data_ptr(), M, H, U.CODES[dtype], U.stream()))
        torch.cuda.synchronize()
        where = f"{M}x{H} offset {off}"
        assert _canaries_intact(hbuf, off, hn) and _canaries_intact(dbuf, off, dn), f"store outside the tensor at {where}"
        U.assert_matches(h.contiguous(), h_ref, dtype, "h, many shapes")
        U.assert_matches(d.contiguous(), d_ref, dtype, "dgu, many shapes", floor=floor)
