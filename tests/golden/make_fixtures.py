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
* ``top_p_cub_order`` — rows for TopPReturnMaskKernel instantiated with a 16-bit DType or float
  (csrc/src/sampling.cu:22-43), where p, the pivots, the width test and every partial sum live in
  half / bfloat16 and the order of the additions is that of cub::BlockReduce with
  BLOCK_REDUCE_WARP_REDUCTIONS (csrc/include/sampling.cuh:54,171-217): each of the 1024 threads
  folds its VEC items left to right, a warp of 32 adds neighbours pairwise (offsets 1, 2, 4, 8,
  16), thread 0 adds the 32 warp results one after the other, and the kernel adds the block sums
  of successive chunks of 1024 * VEC elements. Followed here in exact rational arithmetic with an
  explicit round-to-nearest-even (checked against struct's binary16). Every stored row is one
  whose answer CHANGES under at least one plausible mistake (sums kept exact, a left-to-right
  sum, a tree over a thread's items, a tree over the warp results, a thread summing its items of
  all chunks before one block sum, an unrounded midpoint, an unrounded tolerance), and the rows
  cover all of them and every VEC (8, 4, 2, 1) and one, two and three chunks.
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


# ---- the 16-bit instantiation in CUB's order ------------------------------------------------------
FORMATS = {"f16": (11, -14), "bf16": (8, -126), "f32": (24, -126)}   # significand bits (with the hidden one), e_min


def rne(x, fmt):
    """Round the rational x to the nearest value of the binary format, ties to even."""
    from fractions import Fraction as F
    if x == 0:
        return F(0)
    mant, emin = FORMATS[fmt]
    a = abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    while F(2) ** e > a:
        e -= 1
    while F(2) ** (e + 1) <= a:
        e += 1
    quantum = F(2) ** (max(e, emin) - (mant - 1))
    n = a / quantum
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > F(1, 2) or (rem == F(1, 2) and fl % 2 == 1):
        fl += 1
    return (fl * quantum) * (1 if x > 0 else -1)


def bits_to_frac(b, fmt):
    from fractions import Fraction as F
    if fmt == "f16":
        e, m = (b >> 10) & 31, b & 1023
        return F(m, 1 << 24) if e == 0 else F(1024 + m, 1024) * F(2) ** (e - 15)
    if fmt == "f32":
        e, m = (b >> 23) & 255, b & ((1 << 23) - 1)
        return F(m, 1 << 23) * F(2) ** -126 if e == 0 else F((1 << 23) + m, 1 << 23) * F(2) ** (e - 127)
    e, m = (b >> 7) & 255, b & 127
    return F(m, 128) * F(2) ** -126 if e == 0 else F(128 + m, 128) * F(2) ** (e - 127)


def frac_to_bits(x, fmt):
    from fractions import Fraction as F
    assert x >= 0 and rne(x, fmt) == x
    if x == 0:
        return 0
    mant, emin = FORMATS[fmt]
    e = x.numerator.bit_length() - x.denominator.bit_length()
    while F(2) ** e > x:
        e -= 1
    while F(2) ** (e + 1) <= x:
        e += 1
    bias = 15 if fmt == "f16" else 127
    if e < emin:
        return int(x / F(2) ** (emin - (mant - 1)))
    return ((e + bias) << (mant - 1)) | int((x / F(2) ** e - 1) * (1 << (mant - 1)))


def _check_rounding():
    import random
    import struct
    from fractions import Fraction as F
    rng = random.Random(1)
    for _ in range(4000):
        v = rng.uniform(0, 1) * 2.0 ** rng.randint(-26, 3)
        want = struct.unpack("<e", struct.pack("<e", v))[0]          # the library's binary16
        assert rne(F(v), "f16") == F(want), v
        assert bits_to_frac(struct.unpack("<H", struct.pack("<e", v))[0], "f16") == F(want)
        assert frac_to_bits(F(want), "f16") == struct.unpack("<H", struct.pack("<e", v))[0]
        u = struct.unpack("<I", struct.pack("<f", v))[0]             # bfloat16 = rounded top half
        b = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
        f32 = F(struct.unpack("<f", struct.pack("<f", v))[0])
        assert rne(f32, "bf16") == bits_to_frac(b, "bf16") and frac_to_bits(rne(f32, "bf16"), "bf16") == b
        assert rne(F(v), "f32") == f32 and bits_to_frac(u, "f32") == f32 and frac_to_bits(f32, "f32") == u
    assert rne(F(1, 100000), "f16") == F(168, 1 << 24) and rne(F(3, 1 << 25), "f16") == F(2, 1 << 24)


def _tree(v, add):
    """Pairwise tree over a list whose length is a power of two: what five shuffle-down steps with
    offsets 1, 2, 4, 8, 16 leave in lane 0 of a warp."""
    if len(v) == 1:
        return v[0]
    if not any(v):
        return 0
    return add(_tree(v[:len(v) // 2], add), _tree(v[len(v) // 2:], add))


def cub_block_sums(kept, d, fmt, alt=None):
    """Sum of the entries of `kept` (dict index -> value, everything else 0) as the kernel forms it:
    per chunk of 1024 * VEC elements one cub::BlockReduce, the chunk results added up in order."""
    from fractions import Fraction as F
    from functools import reduce
    from math import gcd
    R = (lambda x: x) if alt == "exact_sums" else (lambda x: rne(x, fmt))
    add = lambda x, y: y if x == 0 else (x if y == 0 else R(x + y))   # adding 0 is exact
    vec = gcd(4 if fmt == "f32" else 8, d)            # 16 / sizeof(DType), sampling.cuh:239
    if alt == "flat_sum":                       # one running sum over the row
        return reduce(add, [kept[i] for i in sorted(kept)], F(0))
    by_chunk = {}
    for i, x in kept.items():
        c, r = divmod(i, 1024 * vec)
        t, j = divmod(r, vec)
        if alt == "chunks_merged":              # a thread sums its items of all chunks first
            c, j = 0, j + vec * (i // (1024 * vec))
        by_chunk.setdefault(c, {}).setdefault(t, {})[j] = x
    total = F(0)
    for c in sorted(by_chunk):
        part = [0] * 1024
        for t, items in by_chunk[c].items():
            n = max(items) + 1
            seq = [items.get(j, 0) for j in range(n)]
            if alt == "thread_tree":
                seq += [0] * (8 * -(-n // 8) - n)
                while len(seq) & (len(seq) - 1):
                    seq.append(0)
                part[t] = _tree(seq, add)
            else:
                part[t] = reduce(add, seq)      # ThreadReduce: left to right from item 0
        warps = [_tree(part[w:w + 32], add) for w in range(0, 1024, 32)]
        block = _tree(warps, add) if alt == "warp_tree" else reduce(add, warps)
        total = add(total, block)
    return F(total)


def cub_top_p(row, d, p_float, high_first, fmt, alt=None):
    """TopPReturnMaskKernel<1024, WARP_REDUCTIONS, VEC, DType> on one row (dict index -> value,
    other entries 0). `alt` names one deliberate mistake. Returns (kept indices, low, iterations)."""
    from fractions import Fraction as F
    p = rne(F(p_float), fmt)
    low, high = F(0), (row.get(0, F(0)) if high_first else max(row.values()))
    eps = F(1, 100000) if alt == "exact_eps" else rne(F(1, 100000), fmt)
    everything = sorted(set(row.values()) | ({F(0)} if len(row) < d else set()))
    iters = 0
    while True:                                  # sampling.cuh:171-217
        iters += 1
        mid = (low + high) / 2 if alt == "exact_mid" else rne(rne(low + high, fmt) / 2, fmt)
        total = cub_block_sums({i: x for i, x in row.items() if x > mid}, d, fmt, alt)
        a = min([high] + [x for x in everything if x > low])
        b = max([low] + [x for x in everything if x <= high])
        if total >= p:
            low = mid
        else:
            high = min(mid, b)
        if not rne(b - a, fmt) > eps or iters > 200:
            break
    return sorted(i for i, x in row.items() if x > low), low, iters


ALTS = ("exact_sums", "flat_sum", "thread_tree", "warp_tree", "chunks_merged", "exact_mid", "exact_eps")


def _random_row(rng, fmt, d, nnz):
    from fractions import Fraction as F
    pos = set(rng.sample(range(d), min(nnz, d)))
    if d > 64:      # crowd a few threads (several terms in a thread's own fold) and a few warps
        for q in rng.sample(sorted(pos), 6):
            pos |= {8 * (q // 8) + k for k in range(8) if 8 * (q // 8) + k < d}
    pos = sorted(pos)
    raw = [rng.paretovariate(1.3) for _ in pos]
    tot = sum(raw)
    row = {i: rne(F(r / tot), fmt) for i, r in zip(pos, raw)}
    return {i: x for i, x in row.items() if x > 0}


def _targeted_rows(fmt):
    """Rows built for the mistakes a random search rarely meets."""
    from fractions import Fraction as F
    if fmt == "f32":
        return []      # the 16-bit rows below live on the grid of binary16 subnormals
    u = F(1, 1 << 24)
    rows = []
    # width of the final bracket exactly fmt(1e-5) = 168 * 2^-24: the loop stops; with an
    # unrounded 1e-5 it would go on
    for big in (F(3, 4), F(1, 2)):
        rows.append(({0: big, 1: F(1, 8), 2: 336 * u, 3: 168 * u}, 8, True))
        rows.append(({0: big, 3: F(1, 16), 5: 1344 * u, 6: 1176 * u, 7: 1008 * u}, 8, False))
    if fmt == "f16":
        # subnormal halving: (0 + 3u) / 2 = 1.5u rounds to 2u, so the elements equal to 2u are
        # not above the first pivot
        rows.append(({0: 3 * u, 1: 2 * u, 2: 2 * u, 3: u}, 4, True))
        rows.append(({0: 5 * u, 1: 3 * u, 2: 2 * u, 5: 2 * u, 6: u}, 7, True))
    return rows


def top_p_cub_order():
    import random
    from fractions import Fraction as F
    _check_rounding()
    out = []
    for fmt in ("f16", "bf16", "f32"):
        rng = random.Random({"f16": 7, "bf16": 8, "f32": 9}[fmt])
        # float: 1e-5 and its float rounding have no float between them, so a bracket width is
        # on the same side of both: that mistake cannot show, the other six can
        missing = set(ALTS) - ({"exact_eps"} if fmt == "f32" else set())
        shapes = [(16, 16), (320, 70), (2048, 90), (12, 12), (8 * 1024 + 24, 140), (10, 10), (7, 7),
                  (3 * 8 * 1024, 200)]
        cands = [(r, d, hf, None) for r, d, hf in _targeted_rows(fmt)]
        tries = 0
        per_shape = {sh: 0 for sh in shapes}
        while tries < 1500 and (missing or min(per_shape.values()) == 0):
            if cands:
                row, d, high_first, _ = cands.pop(0)
                shape = None
            else:
                shape = shapes[tries % len(shapes)]
                d = shape[0]
                row = _random_row(rng, fmt, d, shape[1])
                high_first = rng.random() < 0.5
                if high_first:
                    row[0] = max(row.values())
            tries += 1
            # p = a sum the kernel itself meets at one of its first pivots: that decision is a
            # tie, which another order or width of the sum breaks the other way
            p_choices = [0.5, 0.7, 0.85, 0.9, 0.95]
            lo, hi = F(0), (row[0] if high_first else max(row.values()))
            for _ in range(5):
                mid = rne(rne(lo + hi, fmt) / 2, fmt)
                sub = {i: x for i, x in row.items() if x > mid}
                if sub:
                    s = float(cub_block_sums(sub, d, fmt))
                    if 0 < s <= 1:
                        p_choices += [s, s]
                hi = mid
            for p_float in (p_choices if shape is None else [rng.choice(p_choices)]):
                want = cub_top_p(row, d, p_float, high_first, fmt)
                hit = [a for a in ALTS if cub_top_p(row, d, p_float, high_first, fmt, a) != want]
                new_shape = shape is not None and per_shape[shape] == 0 and hit
                if not (set(hit) & missing) and not new_shape:
                    continue
                missing -= set(hit)
                if shape is not None:
                    per_shape[shape] += 1
                kept, low, iters = want
                out.append({"dtype": fmt, "d": d, "p": p_float, "high": "first" if high_first else "max",
                            "nonzero": [[i, frac_to_bits(x, fmt)] for i, x in sorted(row.items())],
                            "kept": kept, "low_bits": frac_to_bits(low, fmt), "iterations": iters,
                            "differs_under": hit})
                break
        assert not missing and min(per_shape.values()) > 0, (fmt, missing, per_shape)
    return {"source": "csrc/include/sampling.cuh:119-231 with DType = half / nv_bfloat16 / float "
                      "(csrc/src/sampling.cu:22-63), sums in the order of cub::BlockReduce "
                      "BLOCK_REDUCE_WARP_REDUCTIONS, exact rational arithmetic + explicit rounding",
            "rows": out}


def gemv_constant():
    return {"source": "benchmark/efficiency/bench_gemv.py:390-422", "q": 1.0, "nibble": 3,
            "scale": 1.0, "zero": 0.0, "head_dim": 128, "raw_score": 3 * 128}


if __name__ == "__main__":
    out = {"int4_quant": int4_quant(), "top_p_figure": top_p_figure(), "top_p_trace": top_p_trace(),
           "top_p_dyadic": top_p_dyadic(), "top_p_cub_order": top_p_cub_order(),
           "gemv_constant": gemv_constant()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    import re
    text = json.dumps(out, indent=1)
    # innermost lists of numbers on one line each
    text = re.sub(r"\[\s+((?:-?[0-9][0-9.e+-]*,?\s*)+)\]",
                  lambda m: "[" + " ".join(m.group(1).split()) + "]", text)
    with open(path, "w") as f:
        f.write(text + "\n")
    print(path)
