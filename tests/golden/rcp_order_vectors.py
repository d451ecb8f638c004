"""Vectors that tell ``x * (1 / scale)`` from ``x / scale`` in the activation quantizer (the reference multiplies by the
reciprocal, nunchaku/ops/triton/gemm_w4a4.py:1430-1446), with the expected codes derived in exact rational arithmetic.

Each vector is a pair of bf16 values ``(v, gmax)`` placed in one 64-wide group whose other entries are zero, so the group
maximum is ``gmax`` and the fp32 scale is ``fl(gmax / 7)``.  ``fl`` below rounds a rational to fp32 (nearest, ties to
even) without using any floating-point operation, so the two expected codes do not come from the arithmetic under test:
    code_rcp = rne(fl(v * fl(1 / fl(gmax / 7))))        what the reference computes
    code_div = rne(fl(v / fl(gmax / 7)))                what a divide would give
Run this file to search for such pairs again and print them; the tests import ``VECTORS`` and ``expected``."""

import math
from fractions import Fraction as F


def fl(x: F) -> F:
    """x rounded to the nearest fp32 (ties to even); normal range only."""
    if x == 0:
        return F(0)
    s, x = (-1 if x < 0 else 1), abs(x)
    e = math.floor(math.log2(x))
    while F(2) ** e > x:
        e -= 1
    while F(2) ** (e + 1) <= x:
        e += 1
    ulp = F(2) ** (e - 23)
    n, r = divmod(x, ulp)
    n = int(n)
    if r > ulp / 2 or (r == ulp / 2 and n % 2 == 1):
        n += 1
    return s * n * ulp


def rne(x: F) -> int:
    n = math.floor(x)
    r = x - n
    if r > F(1, 2) or (r == F(1, 2) and n % 2 == 1):
        n += 1
    return n


def expected(v: float, gmax: float) -> tuple[int, int]:
    """(code by reciprocal-then-multiply, code by division) for the signed quantizer (qmax = 7)."""
    v, gmax = F(v), F(gmax)
    t = fl(gmax / 7)
    return rne(fl(v * fl(1 / t))), rne(fl(v / t))


# (v, gmax): bf16 values; found by the search below.  The two orders give different codes on every one of them.
VECTORS = [
    (0.12890625, 0.2578125),     # v / scale is exactly 3.5: the divide rounds the tie to 4, the product falls below it
    (0.1591796875, 0.318359375),
    (0.330078125, 0.35546875),
    (-0.1494140625, 0.298828125),
    (0.166015625, 0.33203125),
]


if __name__ == "__main__":
    def bf16s(e_lo, e_hi):
        for e in range(e_lo, e_hi):
            for m in range(128, 256):
                yield F(m) * F(2) ** (e - 7)

    for gmax in bf16s(-2, 3):
        for v in bf16s(-4, 3):
            if v <= gmax:
                a, b = expected(float(v), float(gmax))
                if a != b:
                    print(float(v), float(gmax), a, b)
