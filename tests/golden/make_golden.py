#!/usr/bin/env python3
"""Writes tests/golden/golden_vectors.json: small known-answer vectors for RMSNorm and
SwiGLU, forward and backward.

The reference repository holds no golden vectors for this path (its tests compare against
formulas evaluated at run time), so these are derived here from the DEFINITIONS only, in
50-digit decimal arithmetic, by code that shares nothing with the oracle or the kernels:

  forward   y[r][c] = x[r][c] * w[c] / sqrt(mean_c(x[r][c]^2) + eps)       (test_rmsnorm.py:55-56)
            h[m][j] = g / (1 + exp(-g)) * u                                 (benchmark_swiglu.py:57)
  backward  central finite differences of the scalar L = sum(out * upstream_grad) with step
            1e-20 in 50-digit arithmetic (truncation error ~1e-40): no derivative formula is
            typed in anywhere, so a wrong sign, a dropped term or a transposed index in a
            hand-derived backward pass cannot hide.

Inputs are small dyadic rationals (k/64 or k/8 with |k| <= 255) that fp32, fp16 and bf16 all
represent exactly, so one file serves all three storage types.  Expected values are stored
as the nearest double (repr round-trips).

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
from decimal import Decimal, getcontext
from pathlib import Path

getcontext().prec = 50
H_STEP = Decimal(10) ** -20


class Lcg:
    """Tiny deterministic generator; independent of numpy/torch versions."""

    def __init__(self, seed):
        self.s = seed & 0xFFFFFFFF

    def next(self):
        self.s = (1664525 * self.s + 1013904223) & 0xFFFFFFFF
        return self.s >> 8

    def dyadic(self, denom=64):
        k = self.next() % 511 - 255  # [-255, 255]
        return Decimal(k) / Decimal(denom)


def rmsnorm_fwd(x, w, eps):
    rows, cols = len(x), len(w)
    y, s = [], []
    for r in range(rows):
        ms = sum(v * v for v in x[r]) / Decimal(cols)
        inv = Decimal(1) / (ms + eps).sqrt()
        s.append(inv)
        y.append([x[r][c] * inv * w[c] for c in range(cols)])
    return y, s


def loss_rms(x, w, eps, dy):
    y, _ = rmsnorm_fwd(x, w, eps)
    return sum(y[r][c] * dy[r][c] for r in range(len(x)) for c in range(len(w)))


def rmsnorm_case(seed, rows, cols, eps_str):
    g = Lcg(seed)
    eps = Decimal(eps_str)
    x = [[g.dyadic() for _ in range(cols)] for _ in range(rows)]
    w = [Decimal(1) + g.dyadic(1024) * 4 for _ in range(cols)]   # 1 + k/256: 8-bit significands
    w = [Decimal(int(v * 128)) / 128 for v in w]                  # keep exactly representable in bf16
    dy = [[g.dyadic() for _ in range(cols)] for _ in range(rows)]
    y, s = rmsnorm_fwd(x, w, eps)
    dx = [[None] * cols for _ in range(rows)]
    for r in range(rows):
        for c in range(cols):
            keep = x[r][c]
            x[r][c] = keep + H_STEP
            lp = loss_rms(x, w, eps, dy)
            x[r][c] = keep - H_STEP
            lm = loss_rms(x, w, eps, dy)
            x[r][c] = keep
            dx[r][c] = (lp - lm) / (2 * H_STEP)
    dw = [None] * cols
    for c in range(cols):
        keep = w[c]
        w[c] = keep + H_STEP
        lp = loss_rms(x, w, eps, dy)
        w[c] = keep - H_STEP
        lm = loss_rms(x, w, eps, dy)
        w[c] = keep
        dw[c] = (lp - lm) / (2 * H_STEP)
    f = lambda m: [[float(v) for v in row] for row in m]
    return {
        "rows": rows, "cols": cols, "eps": float(eps),
        "x": f(x), "w": [float(v) for v in w], "dy": f(dy),
        "y": f(y), "inv_rms": [float(v) for v in s], "dx": f(dx), "dw": [float(v) for v in dw],
    }


def swiglu_fwd(gu, H):
    out = []
    for row in gu:
        out.append([row[j] / (Decimal(1) + (-row[j]).exp()) * row[H + j] for j in range(H)])
    return out


def loss_swiglu(gu, H, dh):
    h = swiglu_fwd(gu, H)
    return sum(h[m][j] * dh[m][j] for m in range(len(gu)) for j in range(H))


def swiglu_case(seed, M, H):
    g = Lcg(seed)
    gu = []
    for _ in range(M):
        row = []
        for j in range(2 * H):
            # every fifth gate entry is large in magnitude (k/8, up to +-31.9) to reach both tails
            row.append(g.dyadic(8) if (j < H and j % 5 == 4) else g.dyadic())
        gu.append(row)
    if M * H >= 4:  # exact special points: gate = 0 and the sign pair +-1
        gu[0][0] = Decimal(0)
        gu[0][1] = Decimal(1)
        gu[0][2] = Decimal(-1)
    dh = [[g.dyadic() for _ in range(H)] for _ in range(M)]
    h = swiglu_fwd(gu, H)
    dgu = [[None] * (2 * H) for _ in range(M)]
    for m in range(M):
        for j in range(2 * H):
            keep = gu[m][j]
            gu[m][j] = keep + H_STEP
            lp = loss_swiglu(gu, H, dh)
            gu[m][j] = keep - H_STEP
            lm = loss_swiglu(gu, H, dh)
            gu[m][j] = keep
            dgu[m][j] = (lp - lm) / (2 * H_STEP)
    f = lambda mat: [[float(v) for v in row] for row in mat]
    return {"M": M, "H": H, "gu": f(gu), "dh": f(dh), "h": f(h), "dgu": f(dgu)}


def main():
    data = {
        "comment": "generated by tests/golden/make_golden.py; 50-digit decimal arithmetic, "
                   "finite-difference gradients; inputs exact in fp32/fp16/bf16",
        "rmsnorm": [
            rmsnorm_case(1, 4, 16, "1e-6"),
            rmsnorm_case(2, 3, 8, "1e-5"),
            rmsnorm_case(3, 2, 20, "1e-6"),
            rmsnorm_case(4, 1, 1, "1e-5"),
            rmsnorm_case(5, 5, 33, "1e-3"),
            rmsnorm_case(6, 2, 64, "1e-6"),
        ],
        "swiglu": [
            swiglu_case(11, 4, 16),
            swiglu_case(12, 3, 5),
            swiglu_case(13, 1, 1),
            swiglu_case(14, 2, 24),
        ],
    }
    out = Path(__file__).resolve().parent / "golden_vectors.json"
    out.write_text(json.dumps(data, indent=0))
    print(f"wrote {out} ({out.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
