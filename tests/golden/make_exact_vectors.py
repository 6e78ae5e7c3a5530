"""Writes tests/golden/exact_scan_vectors.json: known-answer vectors in exact rational arithmetic.

The expected values do not come from any implementation of the recurrence.  They come from the
definition of the scan as an explicit sum,

    h(t) = sum_{s<=t} ( prod_{r=s+1..t} a(r) ) * b(s) * x(s),      y(t) = c(t) * h(t),

evaluated with Python fractions, and the gradients of loss = sum(y * dy) from the fact that the
loss is affine in every single scalar input, so that d loss / d v = loss(v + 1) - loss(v)
exactly.  Inputs are small dyadic rationals, exactly representable in fp16, bf16 and fp32.

Run from the repository root:  python tests/golden/make_exact_vectors.py
"""
from __future__ import annotations

import json
import random
from fractions import Fraction
from pathlib import Path

OUT = Path(__file__).resolve().parent / "exact_scan_vectors.json"


def explicit_h(x, a, b, t):
    total = Fraction(0)
    for s in range(t + 1):
        prod = Fraction(1)
        for r in range(s + 1, t + 1):
            prod *= a[r]
        total += prod * b[s] * x[s]
    return total


def column_loss(x, a, b, c, dy):
    return sum(c[t] * explicit_h(x, a, b, t) * dy[t] for t in range(len(x)))


def column_case(x, a, b, c, dy):
    L = len(x)
    h = [explicit_h(x, a, b, t) for t in range(L)]
    y = [c[t] * h[t] for t in range(L)]
    base = column_loss(x, a, b, c, dy)
    grads = {}
    for name, arr in (("dx", x), ("da", a), ("db", b), ("dc", c)):
        g = []
        for t in range(L):
            old = arr[t]
            arr[t] = old + 1
            g.append(column_loss(x, a, b, c, dy) - base)
            arr[t] = old
        grads[name] = g
    return h, y, grads


def dyadic(rng, lo, hi, denom):
    return Fraction(rng.randint(lo * denom, hi * denom), denom)


def make_case(name, B, L, D, seed, a_lo=0, a_hi=1):
    rng = random.Random(seed)
    shape = (B, L, D)

    def tensor(gen):
        return [[[gen() for _ in range(D)] for _ in range(L)] for _ in range(B)]

    x = tensor(lambda: dyadic(rng, -2, 2, 8))
    a = tensor(lambda: dyadic(rng, a_lo, a_hi, 8))
    b = tensor(lambda: dyadic(rng, -1, 1, 8))
    c = tensor(lambda: dyadic(rng, -1, 1, 8))
    dy = tensor(lambda: dyadic(rng, -2, 2, 4))
    out = {k: [[[None] * D for _ in range(L)] for _ in range(B)] for k in ("h", "y", "dx", "da", "db", "dc")}
    for bi in range(B):
        for d in range(D):
            col = lambda ten: [ten[bi][t][d] for t in range(L)]
            h, y, grads = column_case(col(x), col(a), col(b), col(c), col(dy))
            for t in range(L):
                out["h"][bi][t][d] = h[t]
                out["y"][bi][t][d] = y[t]
                for g in ("dx", "da", "db", "dc"):
                    out[g][bi][t][d] = grads[g][t]

    def as_float(ten):
        return [[[float(v) for v in row] for row in mat] for mat in ten]

    def as_text(ten):
        return [[[f"{v.numerator}/{v.denominator}" for v in row] for row in mat] for mat in ten]

    case = {"name": name, "shape": list(shape)}
    for key, ten in (("x", x), ("a", a), ("b", b), ("c", c), ("dy", dy)):
        case[key] = as_float(ten)  # exact: dyadic with small numerators
    for key, ten in out.items():
        case[key] = as_float(ten)           # correctly rounded double of the exact value
        case[key + "_exact"] = as_text(ten)  # the exact rational, for the record
    return case


def main():
    cases = [
        make_case("b1_l6_d2", 1, 6, 2, seed=1),
        make_case("b2_l9_d1", 2, 9, 1, seed=2),
        make_case("b1_l12_d3_growing", 1, 12, 3, seed=3, a_lo=-1, a_hi=2),
        make_case("b3_l1_d2_single_step", 3, 1, 2, seed=4),
    ]
    OUT.write_text(json.dumps({"generator": "tests/golden/make_exact_vectors.py", "cases": cases}, indent=1))
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(cases)} cases)")


if __name__ == "__main__":
    main()
