#!/usr/bin/env python3
"""Writes ``known_answers.json``: the few vectors with known answers that exist for this path.

Nothing here runs or imports the reference or the oracle. The expected values are worked with
plain Python arithmetic from the closed forms the reference's files state, and each is
cross-checked against the literal it is expected to equal:

* ``int4_quant`` — the input vector of twilight/pyimpl/quantize.py:30-48 (the only fixture the
  reference holds for this path; it has no expected output there). Asymmetric 4-bit min/max
  quantisation (quantize.py:4-13): scale = (max - min) / 15, code = round_half_even((x - min) /
  scale) clamped to 0..15, dequantised value = code * scale + min.
* ``top_p_figure`` — the worked example of figures/arch.png: the three largest weights carry
  exactly 0.9, so p = 0.89 keeps the answer away from the rounding of that sum.
* ``top_p_trace`` — a three-element row whose bisection (csrc/include/sampling.cuh:156-231, with
  ``high`` = the first element) is followed by hand: 3 iterations, final low 0.25.
* ``top_p_dyadic`` — rows of powers of two, whose bisection is exact in every arithmetic width: the
  one vector that pins the 16-bit entry point independently of how its sums are ordered.
* ``gemv_constant`` — the constant inputs of benchmark/efficiency/bench_gemv.py:390-422: q = 1,
  every nibble 3, scale 1, zero 0, so every raw score is 3 * 128.
"""
import json
import os

X = [0.31, 0.42, -0.57, 0.23, -1.79, -2.18, 1.90, 4.32, -3.56, 0.78, 0.69, 1.45, 2.84, -2.09, -1.26]


def int4_quant():
    lo, hi = min(X), max(X)
    scale = (hi - lo) / 15
    codes = [min(15, max(0, round((x - lo) / scale))) for x in X]   # round(): half to even
    deq = [c * scale + lo for c in codes]
    assert (lo, hi) == (-3.56, 4.32) and abs(scale - 0.52533334) < 1e-7
    assert codes == [7, 8, 6, 7, 3, 3, 10, 15, 0, 8, 8, 10, 12, 3, 4]
    assert all(abs(d - x) <= scale / 2 + 1e-12 for d, x in zip(deq, X))
    return {"source": "twilight/pyimpl/quantize.py:30-48 (input only)", "x": X, "min": lo, "max": hi,
            "scale": scale, "codes": codes, "dequant": [round(d, 6) for d in deq]}


def top_p_figure():
    w = [0.5, 0.03, 0.005, 0.02, 0.15, 0.005, 0.04, 0.25]
    order = sorted(range(len(w)), key=lambda i: -w[i])
    keep, mass = [], 0.0
    for i in order:                      # textbook nucleus: largest first until the mass reaches p
        if mass >= 0.89:
            break
        keep.append(i)
        mass += w[i]
    assert sorted(keep) == [0, 4, 7] and abs(sum(w) - 1.0) < 1e-12
    return {"source": "figures/arch.png", "weights": w, "p": 0.89, "keep": sorted(keep)}


def top_p_trace():
    probs, p = [0.5, 0.3, 0.2], 0.7
    low, high, iters = 0.0, probs[0], 0
    while True:                          # sampling.cuh:171-217
        iters += 1
        mid = (low + high) / 2
        s = sum(x for x in probs if x > mid)
        a = min([high] + [x for x in probs if x > low])
        b = max([low] + [x for x in probs if x <= high])
        if s >= p:
            low = mid
        else:
            high = min(mid, b)
        if b - a <= 1e-5:
            break
    assert (iters, low) == (3, 0.25)
    return {"source": "csrc/include/sampling.cuh:156-231, high = probs[0]", "probs": probs, "p": p,
            "mask": [1 if x > low else 0 for x in probs], "low": low, "iterations": iters}


def top_p_dyadic():
    """Rows of powers of two: every sum and every midpoint is exact in fp32, fp16 and bf16 alike
    (asserted below: at most 8 significant bits), so the bisection's trace does not depend on the
    width of the arithmetic or on the order of a sum. Token 0 is the row maximum, so both choices
    of the upper bound agree."""
    from fractions import Fraction as F
    rows = [[F(1, 2), F(1, 4), F(1, 8), F(1, 16), F(1, 32), F(1, 32)],
            [F(1, 2), F(1, 8), F(1, 8), F(1, 8), F(1, 16), F(1, 16)],
            [F(1, 4), F(1, 4), F(1, 4), F(1, 8), F(1, 16), F(1, 16)]]
    p = F(7, 8)                     # exact in every width; compared with ">="
    out = []
    for probs in rows:
        assert sum(probs) == 1
        low, high, iters = F(0), probs[0], 0
        while True:                  # sampling.cuh:171-217
            iters += 1
            mid = (low + high) / 2
            n = mid.numerator
            assert n.bit_length() <= 8 and mid.denominator & (mid.denominator - 1) == 0
            s = sum(x for x in probs if x > mid)
            a = min([high] + [x for x in probs if x > low])
            b = max([low] + [x for x in probs if x <= high])
            if s >= p:
                low = mid
            else:
                high = min(mid, b)
            if b - a <= F(1, 100000):
                break
        out.append({"probs": [float(x) for x in probs], "mask": [1 if x > low else 0 for x in probs],
                    "low": float(low), "iterations": iters})
    return {"source": "csrc/include/sampling.cuh:156-231 followed in exact rational arithmetic",
            "p": float(p), "rows": out}


def gemv_constant():
    return {"source": "benchmark/efficiency/bench_gemv.py:390-422", "q": 1.0, "nibble": 3,
            "scale": 1.0, "zero": 0.0, "head_dim": 128, "raw_score": 3 * 128}


if __name__ == "__main__":
    out = {"int4_quant": int4_quant(), "top_p_figure": top_p_figure(), "top_p_trace": top_p_trace(),
           "top_p_dyadic": top_p_dyadic(), "gemv_constant": gemv_constant()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(path)
