"""Exact-rational binary16 arithmetic used to pin the C oracle's soft-float.

Independent of the oracle: values are ``fractions.Fraction``, rounding is done by integer
arithmetic on numerator/denominator (round-to-nearest-even, subnormals, overflow to infinity).
"""
from fractions import Fraction

INF = 0x7C00
SIGN = 0x8000


def h_to_frac(h: int):
    """Exact value of a finite binary16 bit pattern (None for inf/nan)."""
    e, m = (h >> 10) & 0x1F, h & 0x3FF
    if e == 31:
        return None
    v = Fraction(m, 1 << 24) if e == 0 else Fraction(1024 + m, 1) * Fraction(2) ** (e - 25)
    return -v if h & SIGN else v


def is_nan(h):
    return (h & 0x7FFF) > INF


def frac_to_h(v: Fraction, zero_sign: int = 0) -> int:
    """RNE rounding of an exact rational to binary16 bits."""
    if v == 0:
        return zero_sign
    s = SIGN if v < 0 else 0
    a = -v if v < 0 else v
    # exponent E with 2^E <= a < 2^(E+1)
    E = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** E > a:
        E -= 1
    assert Fraction(2) ** E <= a < Fraction(2) ** (E + 1)
    lsb = E - 10 if E >= -14 else -24
    n = a / Fraction(2) ** lsb
    q, r = divmod(n.numerator, n.denominator)
    twice = 2 * r
    if twice > n.denominator or (twice == n.denominator and (q & 1)):
        q += 1
    if lsb == -24:
        return s | q  # q == 1024 is the smallest normal
    e = lsb + 25
    if q == 2048:
        q, e = 1024, e + 1
    if e >= 31:
        return s | INF
    return s | (e << 10) | (q - 1024)


def hmul(a, b):
    fa, fb = h_to_frac(a), h_to_frac(b)
    assert fa is not None and fb is not None
    return frac_to_h(fa * fb, (a ^ b) & SIGN)


def hadd(a, b):
    fa, fb = h_to_frac(a), h_to_frac(b)
    assert fa is not None and fb is not None
    zs = SIGN if (a & SIGN and b & SIGN) else 0
    return frac_to_h(fa + fb, zs)


def hfma(a, b, c):
    fa, fb, fc = h_to_frac(a), h_to_frac(b), h_to_frac(c)
    assert None not in (fa, fb, fc)
    zs = SIGN if (((a ^ b) & SIGN) and (c & SIGN)) else 0
    return frac_to_h(fa * fb + fc, zs)


def from_float(x: float) -> int:
    return frac_to_h(Fraction(x))
