"""Pins of the oracle that need no stored data: closed-form known answers, invariants,
library routines (torch float64 autograd, F.rms_norm, F.silu, gradcheck) and brute force
on tiny inputs.  Each check is chosen so that a plausible slip -- a dropped eps or 1/C, a
wrong sign in the dx correction term, gate/up swapped, a transposed dW -- fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

RNG = np.random.default_rng(1234)


def _rand(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


# ------------------------------------------------------------------- forward known answers

def test_constant_row(oracle):
    c, C, eps = 3.0, 64, 1e-2
    y, s = oracle.rmsnorm_fwd_f64(np.full((2, C), c, np.float32), np.ones(C, np.float32), eps)
    assert s == pytest.approx(1 / math.sqrt(c * c + eps), rel=1e-15)
    assert y == pytest.approx(c / math.sqrt(c * c + eps), rel=1e-15)


def test_one_hot_row(oracle):
    C, a, k, eps = 48, -2.5, 7, 1e-3
    x = np.zeros((1, C), np.float32)
    x[0, k] = a
    w = np.arange(1, C + 1, dtype=np.float32)
    y, s = oracle.rmsnorm_fwd_f64(x, w, eps)
    expect = a * float(w[k]) / math.sqrt(a * a / C + eps)   # catches a missing 1/C
    assert y[0, k] == pytest.approx(expect, rel=1e-15)
    assert np.count_nonzero(y) == 1


def test_zero_row(oracle):
    y, s = oracle.rmsnorm_fwd_f64(np.zeros((3, 10), np.float32), _rand(10), 1e-6)
    assert (y == 0).all()
    assert s == pytest.approx(1e3, rel=1e-15)          # eps^-1/2: catches a dropped eps


def test_scale_invariance_as_eps_vanishes(oracle):
    x, w = _rand(4, 256), _rand(256)
    y1, _ = oracle.rmsnorm_fwd_f64(x, w, 0.0)
    y2, _ = oracle.rmsnorm_fwd_f64(x * np.float32(8.0), w, 0.0)   # power of two: exact scaling
    np.testing.assert_allclose(y1, y2, rtol=1e-14)


def test_f32_and_f64_forward_agree(oracle):
    x, w = _rand(16, 4096), 1 + 0.02 * _rand(4096)
    y32, s32 = oracle.rmsnorm_fwd_f32(x, w, 1e-6)
    y64, s64 = oracle.rmsnorm_fwd_f64(x, w, 1e-6)
    np.testing.assert_allclose(s32, s64, rtol=5e-6)
    np.testing.assert_allclose(y32, y64, rtol=5e-6, atol=1e-7)


# ------------------------------------------------------------------------ library routines

def _torch_formula(x, w, eps):
    # test_rmsnorm.py:55-56
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def test_cpu_reference_configuration_at_full_size(oracle):
    """The CPU-runnable benchmark configuration: x [32,128,4096] fp32 ~N(0,1) from seed 42,
    w = 1 + 0.02 N(0,1), eps = 1e-6, y = x * rsqrt(mean(x^2) + eps) * w.  The literal fp32
    restatement must agree with the PyTorch formula in fp32 within the reference's own
    tolerance (max abs < 1e-4, test_rmsnorm.py:79-81) and with its float64 evaluation."""
    g = torch.Generator().manual_seed(42)
    x = torch.randn((32, 128, 4096), generator=g, dtype=torch.float32)
    w = 1 + 0.02 * torch.randn(4096, generator=g, dtype=torch.float32)
    x2d = x.view(-1, 4096)
    y32, s32 = oracle.rmsnorm_fwd_f32(x2d.numpy(), w.numpy(), 1e-6)
    yt = _torch_formula(x, w, 1e-6).view(-1, 4096).numpy()
    assert y32.shape == (4096, 4096) and s32.shape == (4096,)
    assert np.abs(y32 - yt).max() < 1e-4
    y64 = _torch_formula(x2d.double(), w.double(), 1e-6).numpy()
    np.testing.assert_allclose(y32, y64, rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(s32, torch.rsqrt(x2d.double().pow(2).mean(-1) + 1e-6).numpy(), rtol=2e-6)


@pytest.mark.parametrize("rows,cols", [(5, 33), (8, 128), (3, 4100)])
def test_forward_vs_torch_float64(oracle, rows, cols):
    x, w = _rand(rows, cols), _rand(cols)
    y, _ = oracle.rmsnorm_fwd_f64(x, w, 1e-5)
    yt = _torch_formula(torch.from_numpy(x).double(), torch.from_numpy(w).double(), 1e-5)
    np.testing.assert_allclose(y, yt.numpy(), rtol=1e-12, atol=1e-14)
    yl = F.rms_norm(torch.from_numpy(x).double(), (cols,), torch.from_numpy(w).double(), 1e-5)
    np.testing.assert_allclose(y, yl.numpy(), rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("rows,cols", [(5, 33), (8, 128), (64, 768)])
def test_backward_vs_torch_autograd_float64(oracle, rows, cols):
    x, w, dy = _rand(rows, cols), _rand(cols), _rand(rows, cols)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    wt = torch.from_numpy(w).double().requires_grad_(True)
    (_torch_formula(xt, wt, 1e-5) * torch.from_numpy(dy).double()).sum().backward()
    dx, dw = oracle.rmsnorm_bwd_f64(dy, x, w, 1e-5)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-10, atol=1e-12)
    # the literal fp32 restatement, fed the fp32 inv_rms, agrees to fp32 round-off
    _, s32 = oracle.rmsnorm_fwd_f32(x, w, 1e-5)
    dx32, dw32 = oracle.rmsnorm_bwd_f32(dy, x, w, s32)
    assert np.abs(dx32 - dx).max() / np.abs(dx).max() < 2e-6
    assert np.abs(dw32 - dw).max() / np.abs(dw).max() < 2e-6


def test_gradcheck_of_the_formula_float64():
    """The reference runs gradcheck in fp32 with loose tolerances (test_rmsnorm.py:118-125);
    in float64 the same check is sharp and validates the formula the oracle restates."""
    x = torch.randn(4, 16, dtype=torch.float64, requires_grad=True)
    w = torch.randn(16, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, b: _torch_formula(a, b, 1e-5), (x, w), eps=1e-6, atol=1e-7)


# ------------------------------------------------------------------------ backward identities

def test_dx_orthogonality_identity(oracle):
    """sum_j dx_j x_j = s*A*eps/(mean+eps): vanishes as eps -> 0.  A wrong sign or a missing
    1/C in the correction term breaks it."""
    x, w, dy = _rand(6, 96), _rand(96), _rand(6, 96)
    dx, _ = oracle.rmsnorm_bwd_f64(dy, x, w, 0.0)
    dots = (dx * x.astype(np.float64)).sum(-1)
    assert np.abs(dots).max() < 1e-12
    eps = 0.37
    dx, _ = oracle.rmsnorm_bwd_f64(dy, x, w, eps)
    x64 = x.astype(np.float64)
    mean = (x64 ** 2).mean(-1)
    s = 1 / np.sqrt(mean + eps)
    A = (dy.astype(np.float64) * w.astype(np.float64) * x64).sum(-1)
    np.testing.assert_allclose((dx * x64).sum(-1), s * A * eps / (mean + eps), rtol=1e-11, atol=1e-13)


def test_dx_for_zero_input(oracle):
    w, dy = _rand(32), _rand(3, 32)
    dx, dw = oracle.rmsnorm_bwd_f64(dy, np.zeros((3, 32), np.float32), w, 1e-4)
    np.testing.assert_allclose(dx, 100.0 * dy.astype(np.float64) * w.astype(np.float64), rtol=1e-14)
    assert (dw == 0).all()


def test_dw_brute_force(oracle):
    """dW[j] = sum_r dy[r,j]*x[r,j]*s[r], with plain Python loops (catches a transposed or
    row-summed dW)."""
    rows, cols, eps = 4, 8, 1e-5
    x, w, dy = _rand(rows, cols), _rand(cols), _rand(rows, cols)
    _, dw = oracle.rmsnorm_bwd_f64(dy, x, w, eps)
    for j in range(cols):
        acc = 0.0
        for r in range(rows):
            ms = sum(float(v) ** 2 for v in x[r]) / cols
            acc += float(dy[r, j]) * float(x[r, j]) / math.sqrt(ms + eps)
        assert dw[j] == pytest.approx(acc, rel=1e-13, abs=1e-15)


def test_backward_is_linear_in_dy(oracle):
    x, w, a, b = _rand(5, 40), _rand(40), _rand(5, 40), _rand(5, 40)
    dxa, dwa = oracle.rmsnorm_bwd_f64(a, x, w, 1e-5)
    dxb, dwb = oracle.rmsnorm_bwd_f64(b, x, w, 1e-5)
    dxs, dws = oracle.rmsnorm_bwd_f64((a.astype(np.float64) + b).astype(np.float32), x, w, 1e-5)
    np.testing.assert_allclose(dxs, dxa + dxb, rtol=1e-5, atol=1e-6)   # a+b rounded to fp32
    np.testing.assert_allclose(dws, dwa + dwb, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------------- SwiGLU

def test_swiglu_vs_torch_silu_and_autograd(oracle):
    M, H = 7, 37
    gu, dh = _rand(M, 2 * H) * 3, _rand(M, H)
    t = torch.from_numpy(gu).double().requires_grad_(True)
    out = F.silu(t[:, :H]) * t[:, H:]                    # benchmark_swiglu.py:57
    (out * torch.from_numpy(dh).double()).sum().backward()
    np.testing.assert_allclose(oracle.swiglu_fwd_f64(gu), out.detach().numpy(), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(oracle.swiglu_bwd_f64(dh, gu), t.grad.numpy(), rtol=1e-11, atol=1e-14)


def test_swiglu_known_points(oracle):
    gu = np.array([[0.0, 40.0, -40.0, -1.2784645, 5.0, 6.0, 7.0, 2.0]], np.float32)  # H = 4
    dh = np.array([[3.0, 1.0, 1.0, 1.0]], np.float32)
    h = oracle.swiglu_fwd_f64(gu)[0]
    assert h[0] == 0.0
    assert h[1] == pytest.approx(40.0 * 6.0, rel=1e-15)           # sigmoid(40) = 1 - 4e-18
    assert abs(h[2]) < 40 * 7 * 5e-18                             # far negative tail -> 0
    d = oracle.swiglu_bwd_f64(dh, gu)[0]
    assert d[0] == pytest.approx(3.0 * 5.0 / 2)                   # silu'(0) = 1/2, times dh*up
    assert d[4] == 0.0                                            # d_up = dh*silu(0)
    assert d[1] == pytest.approx(6.0, rel=1e-12)                  # silu'(+inf) = 1
    assert abs(d[3]) < 2e-7                                       # root of silu' near -1.27846


def test_swiglu_halves_not_swapped(oracle):
    gu = np.array([[2.0, 0.0]], np.float32)   # gate = 2, up = 0 -> 0; swapped would give 0 too,
    assert oracle.swiglu_fwd_f64(gu)[0, 0] == 0.0
    gu = np.array([[0.0, 2.0]], np.float32)   # gate = 0, up = 2 -> 0
    assert oracle.swiglu_fwd_f64(gu)[0, 0] == 0.0
    gu = np.array([[1.0, 2.0]], np.float32)   # silu(1)*2, not silu(2)*1
    assert oracle.swiglu_fwd_f64(gu)[0, 0] == pytest.approx(2.0 / (1 + math.exp(-1.0)), rel=1e-15)


# ----------------------------------------------------------------------- rounding helpers

def test_round_to_bf16_is_single_rounding(oracle):
    """1 + 2^-8 + 2^-30 lies just above the midpoint of two bf16 numbers: rounding first to
    fp32 (which drops the 2^-30) and then to bf16 would tie to even (down); one rounding
    goes up."""
    d = np.array([1.0 + 2.0 ** -8 + 2.0 ** -30, 1.0 + 2.0 ** -8, -(1.0 + 3 * 2.0 ** -8)])
    bits = oracle.round_to(d, "bf16")
    assert list(bits) == [0x3F81, 0x3F80, 0xBF82]
    vals = _rand(1000).astype(np.float64)
    t = torch.from_numpy(vals.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (oracle.round_to(vals.astype(np.float32).astype(np.float64), "bf16") == t).all()


def test_ulp_distance(oracle):
    a = np.array([1.0, -1.0, 0.0], np.float32)
    b = np.array([np.nextafter(np.float32(1), np.float32(2)), -1.0, -0.0], np.float32)
    assert list(oracle.ulp_distance(a, b, "fp32")) == [1, 0, 0]
    assert oracle.ulp_distance(np.array([0x3F80], np.uint16), np.array([0x3F82], np.uint16), "bf16")[0] == 2
    assert (oracle.to_f32(np.array([0x3F80, 0xC000], np.uint16), "bf16") == [1.0, -2.0]).all()


# ------------------------------------------------------------------ hypothesis properties

from hypothesis import given, settings, strategies as st  # noqa: E402
from hypothesis.extra import numpy as hnp  # noqa: E402

_small = st.floats(min_value=-8, max_value=8, allow_nan=False, width=32)


@settings(max_examples=60, deadline=None)
@given(hnp.arrays(np.float32, st.tuples(st.integers(1, 5), st.integers(1, 40)), elements=_small))
def test_silu_odd_part_identity(oracle, g):
    """silu(g) - silu(-g) = g, so h(g, u) - h(-g, u) = g*u for any up value: fails if the
    sigmoid is evaluated at the wrong sign or the halves are swapped."""
    u = np.full_like(g, 1.5)
    hp = oracle.swiglu_fwd_f64(np.concatenate([g, u], axis=1))
    hm = oracle.swiglu_fwd_f64(np.concatenate([-g, u], axis=1))
    np.testing.assert_allclose(hp - hm, g.astype(np.float64) * 1.5, rtol=1e-12, atol=1e-12)


@settings(max_examples=60, deadline=None)
@given(hnp.arrays(np.float32, st.tuples(st.integers(1, 4), st.integers(2, 48)), elements=_small),
       st.integers(0, 10 ** 6))
def test_rmsnorm_row_has_unit_mean_square(oracle, x, seed):
    """With w = 1 and eps = 0 every output row has mean square exactly 1 (rows of zeros aside)."""
    x = x + np.float32(0.125) * np.float32(1 + seed % 3)          # keep rows away from all-zero
    y, s = oracle.rmsnorm_fwd_f64(x, np.ones(x.shape[1], np.float32), 0.0)
    keep = np.abs(x).max(-1) > 0
    np.testing.assert_allclose((y[keep] ** 2).mean(-1), 1.0, rtol=1e-12)


@settings(max_examples=40, deadline=None)
@given(hnp.arrays(np.float32, st.tuples(st.integers(1, 4), st.integers(2, 32)), elements=_small))
def test_rmsnorm_gradient_matches_finite_difference(oracle, x):
    """Directional derivative of L = sum(y*dy) along a fixed direction, by central differences
    in double precision, against <dx, direction> from the oracle's backward."""
    rows, cols = x.shape
    rng = np.random.default_rng(rows * 100 + cols)
    w = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    d = rng.standard_normal((rows, cols))
    eps = 1e-2

    def loss(xx):
        xx = np.asarray(xx, np.float64)
        s = 1 / np.sqrt((xx ** 2).mean(-1, keepdims=True) + eps)
        return float((xx * s * w * dy).sum())

    h = 1e-6
    fd = (loss(x + h * d) - loss(x - h * d)) / (2 * h)
    dx, _ = oracle.rmsnorm_bwd_f64(dy, x, w, eps)
    assert fd == pytest.approx(float((dx * d).sum()), rel=1e-5, abs=1e-6)
