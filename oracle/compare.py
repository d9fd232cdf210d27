"""Comparison rules of the parity tests (test infrastructure, like the rest of this package).

  fp32 outputs       |got - ref| <= 1e-5 * |ref|
  fp16/bf16 outputs  at most 1 unit in the last place away from the double-precision answer
                     rounded once to the output type
  cancellation floor dx and d_gate are sums of terms of either sign:
                       dx[r,c] = s*dy*w  -  sum_j x[r,c]*(s^3/C)*dy[r,j]*w[j]*x[r,j]
                     Where the terms nearly cancel, no fp32 evaluation (the reference's
                     included) resolves the result to 1 ulp of itself; what fp32 arithmetic
                     does guarantee is the forward error bound of a computed sum, a few ulps
                     of the sum of the terms' magnitudes.  An element that misses the rule
                     above therefore still passes when |got - ref| <= 4 * 2^-24 * floor, floor
                     being that sum of magnitudes -- but such elements are counted, and the
                     tensor fails when they are more than FLOOR_SHARE_CAP of its elements plus
                     the number of elements at which the literal fp32 restatement of the
                     reference's own arithmetic needs the floor as well (how many elements
                     cancel that deeply is a property of the data).  A systematic error hiding
                     behind the floor would show as an excess.  The one exception is asked for
                     by name (`every_element_cancels`): rows of a single column, where
                     dx = s*dy*w*eps/(x^2+eps) is nothing but the difference of two equal
                     terms; there every element is held to the floor bound and none to 1 ulp.
  dW                 on the fp32 buffer, scale-aware: max|got - ref| / max|ref| <= 1e-3 and
                     ||got - ref||_2 / ||ref||_2 <= 1e-3
"""
from __future__ import annotations

import numpy as np

from .oracle import round_to, to_f32, ulp_distance

FP32_ULP = 2.0 ** -24
FLOOR_FACTOR = 4.0
# largest share of a tensor's elements that may pass through the cancellation floor only
FLOOR_SHARE_CAP = {"fp32": 5e-3, "fp16": 1e-4, "bf16": 1e-4}

# what -> [elements compared, elements that passed through the floor only, worst err / (2^-24 * floor),
#          elements at which the reference's own fp32 arithmetic needs the floor]
STATS: dict = {}


class Floor:
    """The cancellation floor of a tensor (`bound` = sum of the magnitudes of its terms) and,
    optionally, what the literal fp32 restatement of the reference arithmetic gives for the
    same inputs (`ref32`), which sets how many elements may be expected to need the floor."""

    def __init__(self, bound, ref32=None):
        self.bound = np.asarray(bound, dtype=np.float64)
        self.ref32 = None if ref32 is None else np.asarray(ref32, dtype=np.float32)


def _misses(g64, g_store, ref64, dtype):
    """|error|, the elements that miss the output rule, and the ulp distances (2-byte types)."""
    err = np.abs(g64 - ref64)
    if dtype == "fp32":
        return err, err > 1e-5 * np.abs(ref64) + 1e-37, None
    ulps = ulp_distance(g_store, round_to(ref64, dtype), dtype)
    return err, ulps > 1, ulps


def storage_view(t, dtype: str) -> np.ndarray:
    """float32 / float16 arrays as they are, uint16 bit patterns for bf16 (from a torch tensor)."""
    import torch

    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def assert_matches(got, ref64, dtype: str, what: str, floor=None, every_element_cancels=False):
    """Apply the output rule to one tensor (`got`: torch tensor of the storage type; `floor`:
    a Floor, or just the array of bounds).  Returns how many elements needed the floor.
    `every_element_cancels`: the caller states that the tensor consists of differences of
    equal terms only (one-column rows), so no share of it is expected within 1 ulp."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    g_store = storage_view(got, dtype)
    g64 = to_f32(g_store, dtype).astype(np.float64)
    assert g64.shape == ref64.shape, f"{what}: shape {g64.shape} vs {ref64.shape}"
    assert np.isfinite(g64).all(), f"{what}: non-finite values in the output"
    err, miss, ulps = _misses(g64, g_store, ref64, dtype)
    if dtype == "fp32":
        detail = lambda i: f"rel err {err[i] / max(abs(ref64[i]), 1e-300):.3e}"
    else:
        detail = lambda i: f"{ulps[i]} ulp"
    bad = miss
    n_floor, worst, n_expected = 0, 0.0, 0
    if floor is not None:
        ref32 = floor.ref32 if isinstance(floor, Floor) else None
        floor = floor.bound if isinstance(floor, Floor) else np.asarray(floor, dtype=np.float64)
        bad = miss & (err > FLOOR_FACTOR * FP32_ULP * floor)
        via_floor = miss & ~bad
        n_floor = int(via_floor.sum())
        if n_floor:
            worst = float((err[via_floor] / (FP32_ULP * floor[via_floor])).max())
        if ref32 is not None and n_floor:
            # the reference arithmetic in fp32, rounded once to the storage type, under the same rule
            r_store = ref32 if dtype == "fp32" else round_to(ref32.astype(np.float64), dtype)
            r64 = to_f32(r_store, dtype).astype(np.float64)
            _, r_miss, _ = _misses(r64, r_store, ref64, dtype)
            n_expected = int(r_miss.sum())
    rec = STATS.setdefault(f"{what} [{dtype}]", [0, 0, 0.0, 0])
    rec[0] += miss.size
    rec[1] += n_floor
    rec[2] = max(rec[2], worst)
    rec[3] += n_expected
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, err, -1.0)), err.shape)
        raise AssertionError(
            f"{what} [{dtype}]: {int(bad.sum())} of {bad.size} elements out of tolerance; worst at {idx}: "
            f"got {g64[idx]!r}, ref {ref64[idx]!r}, {detail(idx)}")
    # small tensors: allow a handful of elements whatever the share
    if not every_element_cancels and n_floor > max(4, FLOOR_SHARE_CAP[dtype] * miss.size) + n_expected:
        raise AssertionError(
            f"{what} [{dtype}]: {n_floor} of {miss.size} elements pass only through the cancellation floor "
            f"(cap {FLOOR_SHARE_CAP[dtype]:.0e} of the elements + the {n_expected} at which the reference's "
            f"fp32 arithmetic needs it too): too many for rounding alone")
    return n_floor


def assert_dw(dw_f32, ref64, what="dW"):
    got = dw_f32.detach().cpu().numpy().astype(np.float64)
    ref64 = np.asarray(ref64, dtype=np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite"
    scale = max(np.abs(ref64).max(), 1e-300)
    e_max = np.abs(got - ref64).max() / scale
    e_l2 = np.linalg.norm(got - ref64) / max(np.linalg.norm(ref64), 1e-300)
    assert e_max <= 1e-3 and e_l2 <= 1e-3, f"{what}: max-scaled err {e_max:.3e}, l2 err {e_l2:.3e}"
    return e_max, e_l2


def dx_floor(x, dy, w, s):
    """Sum of the magnitudes of the terms dx is made of (see the module docstring)."""
    x, dy, w, s = (np.asarray(a, dtype=np.float64) for a in (x, dy, w, s))
    cols = x.shape[1]
    gwx = np.abs(dy * w * x).sum(-1, keepdims=True)
    return np.abs(s[:, None] * dy * w) + np.abs(x) * (s[:, None] ** 3 / cols) * gwx


def swiglu_floor(dh, gu):
    """The same for [d_gate | d_up]: d_gate = dh*u*sig*(1 + g*(1-sig)) cancels for g < 0;
    d_up is a plain product (floor 0)."""
    dh, gu = np.asarray(dh, dtype=np.float64), np.asarray(gu, dtype=np.float64)
    H = gu.shape[1] // 2
    g, u = gu[:, :H], gu[:, H:]
    with np.errstate(over="ignore"):
        sig = 1.0 / (1.0 + np.exp(-g))
    base = np.abs(dh * u * sig)
    return np.concatenate([base * (1.0 + np.abs(g) * (1.0 - sig)), np.zeros_like(base)], axis=1)


def stats_lines():
    lines = []
    for key, (n, nf, worst, nexp) in sorted(STATS.items()):
        if nf:
            lines.append(f"{key}: {nf} of {n} elements ({nf / n:.2e}) passed through the cancellation floor only "
                         f"(the reference's fp32 arithmetic needs it at {nexp}); "
                         f"worst error there {worst:.2f} x 2^-24 x sum|terms| (limit {FLOOR_FACTOR:.0f})")
    return lines
