"""Exact-rational model of the reference quantizer's binary32 arithmetic (asymmetric_quant.py:80-104):
every operation is evaluated exactly with fractions and then rounded to the nearest binary32 value,
independently of numpy, torch and the C oracle.  Shared by tests/test_oracle_quant.py and by
tests/golden/make_golden.py, which derives the committed known-answer rows from it."""
import math
from fractions import Fraction


def rn32(fr: Fraction) -> Fraction:
    """Round an exact rational to the nearest binary32 value (ties to even), exactly."""
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = math.floor(math.log2(a)) if a >= 1 else -math.ceil(math.log2(1 / a))
    while Fraction(2) ** e > a:
        e -= 1
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -126)                      # subnormals share the exponent of the smallest normal
    ulp = Fraction(2) ** (e - 23)
    q = a / ulp
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    out = n * ulp
    assert out < Fraction(2) ** 128
    return sign * out


def roundf_exact(fr: Fraction) -> int:
    """C roundf on an exact value: nearest integer, ties away from zero."""
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    n = a.numerator // a.denominator
    if a - n >= Fraction(1, 2):
        n += 1
    return sign * n


def quant_row_exact(row):
    """asymmetric_quant.py:80-104 with every fp32 operation modelled as exact-then-round."""
    xs = [Fraction(float(v)) for v in row]
    mn, mx = min(xs), max(xs)
    scale = rn32(rn32(mx - mn) / 255)
    if scale == 0:
        scale = Fraction(1)
    zpf = rn32(Fraction(-128) - rn32(mn / scale))
    zp = max(-128, min(127, roundf_exact(zpf)))
    codes = [max(-128, min(127, roundf_exact(rn32(rn32(x / scale) + zp)))) for x in xs]
    return codes, scale, zp
