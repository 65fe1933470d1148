"""Exact emulation of IEEE-754 binary32 arithmetic with Python fractions.

Used to pin the *order* of the oracle's floating-point sums: every operation is
computed exactly as a rational number and rounded once to binary32 (round to
nearest, ties to even), which is what the hardware add / multiply / fused
multiply-add do.  Only normal-range values are supported (enough for the tests).
"""
from fractions import Fraction

import numpy as np


def to_frac(x):
    return Fraction(float(np.float32(x)))


def round32(q):
    """Round the rational q to the nearest binary32 value (ties to even)."""
    if q == 0:
        return Fraction(0)
    sign = -1 if q < 0 else 1
    a = -q if q < 0 else q
    # exponent e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    elif Fraction(2) ** (e + 1) <= a:
        e += 1
    assert -126 <= e <= 127, "value outside the normal binary32 range"
    scale = Fraction(2) ** (e - 23)
    m = a / scale                      # in [2^23, 2^24)
    fl = m.numerator // m.denominator
    rem = m - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        fl += 1
    return sign * fl * scale


def add(x, y):
    return round32(x + y)


def sub(x, y):
    return round32(x - y)


def mul(x, y):
    return round32(x * y)


def fma(x, y, z):
    return round32(x * y + z)


def as_f32(q):
    return np.float32(float(q))
