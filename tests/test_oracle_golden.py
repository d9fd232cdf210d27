"""The C oracle against the committed golden vectors (tests/golden/golden_vectors.json:
50-digit decimal arithmetic, gradients by finite differences -- no derivative formula
shared with the oracle).  The *_f64 oracle must agree to double-precision round-off; the
literal *_f32 restatement to fp32 round-off."""
import numpy as np
import pytest


def _rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    scale = max(np.abs(b).max(), 1e-300)
    return np.abs(a - b).max() / scale


@pytest.mark.parametrize("idx", range(6))
def test_rmsnorm_f64_matches_golden(oracle, golden, idx):
    c = golden["rmsnorm"][idx]
    x, w, dy = (np.array(c[k], np.float32) for k in ("x", "w", "dy"))
    assert (x.astype(np.float64) == np.array(c["x"])).all()  # inputs are exact in fp32
    y, s = oracle.rmsnorm_fwd_f64(x, w, c["eps"])
    np.testing.assert_allclose(y, np.array(c["y"]), rtol=1e-13, atol=1e-300)
    np.testing.assert_allclose(s, np.array(c["inv_rms"]), rtol=1e-13)
    dx, dw = oracle.rmsnorm_bwd_f64(dy, x, w, c["eps"])
    assert _rel(dx, c["dx"]) < 1e-13
    assert _rel(dw, c["dw"]) < 1e-13


@pytest.mark.parametrize("idx", range(6))
def test_rmsnorm_f32_matches_golden(oracle, golden, idx):
    c = golden["rmsnorm"][idx]
    x, w, dy = (np.array(c[k], np.float32) for k in ("x", "w", "dy"))
    y, s = oracle.rmsnorm_fwd_f32(x, w, c["eps"])
    assert _rel(y, c["y"]) < 1e-6
    assert _rel(s, c["inv_rms"]) < 1e-6
    dx, dw = oracle.rmsnorm_bwd_f32(dy, x, w, s)
    # dx is a difference of two terms of size |s*dy*w| (they cancel almost fully in the
    # 1x1 case), so fp32 round-off is measured against that size
    scale = np.abs(s[:, None] * dy * w).max()
    assert np.abs(dx - np.array(c["dx"])).max() / scale < 2e-6
    assert _rel(dw, c["dw"]) < 2e-6


@pytest.mark.parametrize("idx", range(4))
def test_swiglu_matches_golden(oracle, golden, idx):
    c = golden["swiglu"][idx]
    gu, dh = np.array(c["gu"], np.float32), np.array(c["dh"], np.float32)
    h = oracle.swiglu_fwd_f64(gu)
    np.testing.assert_allclose(h, np.array(c["h"]), rtol=1e-13, atol=1e-300)
    d = oracle.swiglu_bwd_f64(dh, gu)
    # relative to the largest gradient: entries in the far negative tail are ~1e-13 small
    assert _rel(d, c["dgu"]) < 1e-13
    np.testing.assert_allclose(d, np.array(c["dgu"]), rtol=1e-9, atol=1e-18)
    assert _rel(oracle.swiglu_fwd_f32(gu), c["h"]) < 1e-6
    assert _rel(oracle.swiglu_bwd_f32(dh, gu), c["dgu"]) < 1e-6


def test_golden_layout_gate_first(golden):
    """[gate | up] order: with gate = 0 the output is 0 whatever `up` holds, and the
    gradient with respect to gate is dh*up/2 (silu'(0) = 1/2)."""
    c = golden["swiglu"][0]
    H = c["H"]
    assert c["gu"][0][0] == 0.0 and c["h"][0][0] == 0.0
    assert c["dgu"][0][0] == pytest.approx(c["dh"][0][0] * c["gu"][0][H] / 2, rel=1e-12)
    assert c["dgu"][0][H] == pytest.approx(0.0, abs=1e-18)
