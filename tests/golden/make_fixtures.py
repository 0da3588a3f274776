"""Writes the golden fixtures in this directory.

Everything here is derived from definitions, not from the oracle and not from
the product: the OCP 8-bit float formats are evaluated with exact rationals,
integer GEMMs with Python ints, and the reference's own hand vectors are
transcribed as data (inputs and expected outputs only).

Run:  python tests/golden/make_fixtures.py
"""

from __future__ import annotations

import json
import os
import random
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


# ---------------------------------------------------------------------------
# OCP fp8 definitions, exact
# ---------------------------------------------------------------------------

def decode(code: int, ebits: int, mbits: int, bias: int, fn: bool):
    """Value of an 8-bit code as Fraction, or 'nan' / 'inf' / '-inf'."""
    sign = -1 if code >> 7 else 1
    e = (code >> mbits) & ((1 << ebits) - 1)
    m = code & ((1 << mbits) - 1)
    top = (1 << ebits) - 1
    if fn:
        if e == top and m == (1 << mbits) - 1:
            return "nan"
    elif e == top:
        return "nan" if m else ("inf" if sign > 0 else "-inf")
    if e == 0:
        return sign * Fraction(m) * Fraction(2) ** (1 - bias - mbits)
    return sign * Fraction((1 << mbits) | m) * Fraction(2) ** (e - bias - mbits)


E4M3 = dict(ebits=4, mbits=3, bias=7, fn=True)
E5M2 = dict(ebits=5, mbits=2, bias=15, fn=False)


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def f32_from_bits(b: int) -> float:
    return struct.unpack("<f", struct.pack("<I", b))[0]


def f32_next(x: float, up: bool) -> float:
    b = f32_bits(x)
    assert x > 0
    return f32_from_bits(b + 1 if up else b - 1)


def cast_rne(x: float, fmt: dict) -> int:
    """Round-to-nearest-even cast of a finite float to a code, by brute force
    over all finite codes with exact rationals. Overflow follows the unbounded-
    exponent rule: values that round (RNE, as if the exponent range continued)
    to a magnitude above the finite max become NaN (fn) or inf (IEEE-like)."""
    fx = Fraction(x)
    sign_bit = 0x80 if (x < 0 or (x == 0 and str(x).startswith("-"))) else 0
    mag = abs(fx)
    finite = []
    for c in range(128):
        v = decode(c, **fmt)
        if isinstance(v, Fraction):
            finite.append((v, c))
    finite.sort()
    vmax, cmax = finite[-1]
    # spacing of the top binade
    ulp_top = vmax - finite[-2][0]
    overflow_boundary = vmax + ulp_top / 2
    mbits = fmt["mbits"]
    if mag > overflow_boundary or (mag == overflow_boundary and (cmax & 1)):
        # tie at the boundary goes to the even neighbour: the (non-existent) next
        # value has an even mantissa, so a tie rounds up when cmax is odd.
        if fmt["fn"]:
            return sign_bit | 0x7F
        return sign_bit | (((1 << fmt["ebits"]) - 1) << mbits)
    if mag == overflow_boundary:
        return sign_bit | cmax
    best = None
    for v, c in finite:
        d = abs(mag - v)
        if best is None or d < best[0] or (d == best[0] and (c & 1) == 0 and (best[1] & 1)):
            best = (d, c)
    return sign_bit | best[1]


def cast_vectors(fmt: dict):
    """Inputs chosen so that a wrong rounding mode, a flushed subnormal or a wrong
    overflow rule fails: every midpoint between adjacent finite codes (a tie), its
    float32 neighbours, every code value itself, half the smallest subnormal and
    its neighbours, and the overflow boundary and its neighbours."""
    vals = []
    finite = sorted(
        (decode(c, **fmt), c) for c in range(128) if isinstance(decode(c, **fmt), Fraction)
    )
    for (v0, _), (v1, _) in zip(finite, finite[1:]):
        mid = float((v0 + v1) / 2)
        vals += [mid, f32_next(mid, True), f32_next(mid, False)]
    vals += [float(v) for v, _ in finite]
    vmax = finite[-1][0]
    ulp_top = vmax - finite[-2][0]
    ob = float(vmax + ulp_top / 2)
    vals += [ob, f32_next(ob, True), f32_next(ob, False), float(vmax) * 2, 1e30]
    out = []
    for v in vals:
        for s in (1.0, -1.0):
            x = s * v
            if x == 0 and s < 0:
                x = -0.0
            out.append([f32_bits(x), cast_rne(x, fmt)])
    return out


def table(fmt: dict):
    out = []
    for c in range(256):
        v = decode(c, **fmt)
        if isinstance(v, str):
            out.append(v)
        elif v == 0 and c >> 7:
            out.append((-0.0).hex())  # Fraction drops the sign of zero
        else:
            out.append(float(v).hex())
    return out


# ---------------------------------------------------------------------------
# Integer GEMM and per-row int8 quantization, exact
# ---------------------------------------------------------------------------

def int8_cases():
    cases = []
    for seed, (m, n, k) in enumerate([(1, 1, 1), (3, 5, 7), (17, 9, 33), (16, 16, 64), (2, 3, 130)]):
        r = random.Random(1000 + seed)
        a = [[r.randint(-127, 127) for _ in range(k)] for _ in range(m)]
        b = [[r.randint(-127, 127) for _ in range(k)] for _ in range(n)]
        acc = [[sum(a[i][p] * b[j][p] for p in range(k)) for j in range(n)] for i in range(m)]
        cases.append({"m": m, "n": n, "k": k, "a": a, "b": b, "acc": acc})
    # worst-case magnitude: every product is 127*127 (or -127*127)
    k = 4096
    a = [[127] * k, [-127] * k]
    b = [[127] * k, [-127] * k, [127, -127] * (k // 2)]
    acc = [[sum(x * y for x, y in zip(ar, br)) for br in b] for ar in a]
    cases.append({"m": 2, "n": 3, "k": k, "a": a, "b": b, "acc": acc})
    return cases


def bf16_round(x: float) -> float:
    b = f32_bits(np.float32(x).item())
    lsb = (b >> 16) & 1
    b = (b + 0x7FFF + lsb) & 0xFFFF0000
    return f32_from_bits(b)


def rne_int(fr: Fraction) -> int:
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        return fl + 1
    return fl


def int8_quant_cases():
    """Rows of bf16 values; s = fl32(amax/127); q = clamp(rne(fl32(x/s)), +-127)."""
    cases = []
    r = random.Random(77)
    rows = [
        [bf16_round(r.gauss(0, 1)) for _ in range(24)],
        [bf16_round(r.gauss(0, 0.02)) for _ in range(24)],
        [0.0] * 8,                                 # all-zero row -> s = 1e-12/127
        [127.0, -63.5, 62.5, 0.5, 1.5, 2.5, -0.5, -1.5],  # s = 1: exact ties
        [254.0, 1.0, 3.0, 5.0, -1.0, -3.0, 253.0, -254.0],  # s = 2: ties at odd
    ]
    for row in rows:
        amax = max(abs(v) for v in row)
        amax = max(np.float32(amax), np.float32(1e-12))
        s = np.float32(amax) / np.float32(127.0)
        q = []
        for v in row:
            d = np.float32(v) / s  # correctly rounded fp32 division
            qi = rne_int(Fraction(float(d)))
            q.append(max(-127, min(127, qi)))
        cases.append({"x": row, "scale_bits": f32_bits(float(s)), "q": q})
    return cases


# ---------------------------------------------------------------------------
# fp8 GEMM (per-tensor and 128-block) on small shapes, exact rationals
# ---------------------------------------------------------------------------

def fp8_gemm_cases():
    cases = []
    r = random.Random(5)
    finite_codes = [c for c in range(256) if isinstance(decode(c, **E4M3), Fraction)]
    for (m, n, k) in [(2, 3, 8), (4, 2, 128)]:
        a = [[r.choice(finite_codes) for _ in range(k)] for _ in range(m)]
        b = [[r.choice(finite_codes) for _ in range(k)] for _ in range(n)]
        sa, sb = 0.75, 1.5
        exact = [[float(sum(decode(a[i][p], **E4M3) * decode(b[j][p], **E4M3) for p in range(k))
                        * Fraction(sa) * Fraction(sb)) for j in range(n)] for i in range(m)]
        cases.append({"m": m, "n": n, "k": k, "a": a, "b": b, "sa": sa, "sb": sb, "exact": exact})
    return cases


def block128_cases():
    r = random.Random(9)
    # small-magnitude codes keep the exact sums well inside fp32 range
    codes = [c for c in range(256) if isinstance(decode(c, **E4M3), Fraction)
             and abs(decode(c, **E4M3)) <= 16]
    m, n, k = 3, 130, 256
    kb, nb = k // 128, 2
    a = [[r.choice(codes) for _ in range(k)] for _ in range(m)]
    b = [[r.choice(codes) for _ in range(k)] for _ in range(n)]
    sa = [[float(np.float32(r.uniform(0.01, 2.0))) for _ in range(kb)] for _ in range(m)]
    sb = [[float(np.float32(r.uniform(0.01, 2.0))) for _ in range(kb)] for _ in range(nb)]
    exact = []
    for i in range(m):
        row = []
        for j in range(n):
            tot = Fraction(0)
            for q in range(kb):
                part = sum(decode(a[i][p], **E4M3) * decode(b[j][p], **E4M3)
                           for p in range(q * 128, q * 128 + 128))
                tot += part * Fraction(sa[i][q]) * Fraction(sb[j // 128][q])
            row.append(float(tot))
        exact.append(row)
    return [{"m": m, "n": n, "k": k, "a": a, "b": b, "sa": sa, "sb": sb, "exact": exact}]


# ---------------------------------------------------------------------------
# The reference's own hand vectors for this path (data only)
# ---------------------------------------------------------------------------

REFERENCE_KATS = {
    "source": "tests/extension/test_fp8_mma.py",
    "mm_fp8_cpu": {  # :273-280
        "a8": [[1.0, 2.0]], "b8": [[3.0, 4.0]], "sa": 2.0, "sb": 0.5, "out_bf16": [[11.0]],
    },
    "mm_fp8_fp8_out_cpu": {  # :283-293
        "a8": [[1.0, 2.0]], "b8": [[3.0, 4.0]], "sa": 2.0, "sb": 0.5, "out_scale": 0.25,
        "out_e4m3": [[2.75]],
    },
    "recipe": [  # :206-222  (history, fmt, margin, expected scale)
        {"hist": [1.0, 2.0, 0.5], "fmt": "e4m3", "margin": 0, "scale": 2.0 / 448.0},
        {"hist": [1.0, 2.0, 0.5], "fmt": "e4m3", "margin": 2, "scale": 2.0 / 448.0 / 4.0},
        {"hist": [0.25], "fmt": "e4m3", "margin": 0, "scale": 0.25 / 448.0},
        {"hist": [0.25], "fmt": "e5m2", "margin": 0, "scale": 0.25 / 57344.0},
    ],
    "meta_update": {"amax": 4.0, "scale": 4.0 / 448.0},  # :251-259
    "quantize_scale": 0.5,  # :65-77, :262-270: x8 == (x/0.5).to(e4m3fn) bit-exactly
    "ragged_shapes": [[16, 8, 32], [17, 9, 33], [31, 15, 64], [32, 48, 96]],  # :45
    "fwd_bwd_shape": [19, 13, 37],  # :88-116 (seed 7, with bias)
    "tolerances": {"small": {"atol": 0.125, "rtol": 0.01},       # :61
                   "k4096_vs_f64": {"atol": 6.0, "rtol": 0.05},  # :163
                   "vs_scaled_mm": {"atol": 2.0, "rtol": 0.01}},  # :169-174
}


def main():
    fixtures = {
        "fp8_codes.json": {
            "e4m3fn_decode": table(E4M3),
            "e5m2_decode": table(E5M2),
            "e4m3fn_cast": cast_vectors(E4M3),
            "e5m2_cast": cast_vectors(E5M2),
        },
        "int8_small.json": {"gemm": int8_cases(), "quantize_rows": int8_quant_cases()},
        "fp8_gemm_small.json": {"per_tensor": fp8_gemm_cases(), "block128": block128_cases()},
        "reference_kats.json": REFERENCE_KATS,
    }
    for name, obj in fixtures.items():
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(obj, f, separators=(",", ":"))
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
