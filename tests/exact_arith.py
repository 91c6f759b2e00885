"""Exact rational arithmetic used to pin the oracle on tiny inputs: every floating-point operation of
the reference is re-derived as "exact rational result, then one IEEE round-to-nearest-even", with
Python integers and Fractions only (no float arithmetic, no shared code with the oracle)."""

from fractions import Fraction


def _floor_log2(a: Fraction) -> int:
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    elif Fraction(2) ** (e + 1) <= a:
        e += 1
    return e


def round_to_format(v: Fraction, precision: int, emin: int) -> Fraction:
    """Nearest value with `precision` significand bits and minimum normal exponent `emin`
    (gradual underflow below it), ties to even.  No overflow handling: callers keep values in range."""
    if v == 0:
        return Fraction(0)
    sign = -1 if v < 0 else 1
    a = abs(v)
    e = max(_floor_log2(a), emin)
    ulp = Fraction(2) ** (e - precision + 1)
    q = a / ulp
    n = q.numerator // q.denominator
    r = q - n
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return sign * n * ulp


def rn_f32(v: Fraction) -> Fraction:
    return round_to_format(v, 24, -126)


def rn_bf16(v: Fraction) -> Fraction:
    return round_to_format(v, 8, -126)


def rn_e4m3(v: Fraction) -> Fraction:
    """Value of the e4m3fn code v rounds to (|result| <= 448 assumed)."""
    return round_to_format(v, 4, -6)


def rne_int(v: Fraction) -> int:
    n = v.numerator // v.denominator
    r = v - n
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return n


def e4m3_code(v: Fraction, negative_zero: bool = False) -> int:
    """e4m3fn byte of an exactly representable value."""
    sign = 0x80 if (v < 0 or (v == 0 and negative_zero)) else 0
    a = abs(v)
    if a == 0:
        return sign
    if a < Fraction(1, 64):
        k = a * 512
        assert k.denominator == 1
        return sign | int(k)
    e = _floor_log2(a)
    m = (a / Fraction(2) ** e - 1) * 8
    assert m.denominator == 1 and 0 <= m < 8 and -6 <= e <= 8
    return sign | ((e + 7) << 3) | int(m)


F32_ONE_SEVENTH = rn_f32(Fraction(1, 7))
F32_1EM5 = rn_f32(Fraction(1, 100000))
F32_1EM10 = rn_f32(Fraction(1, 10 ** 10))
BF16_1EM12 = rn_bf16(Fraction(1, 10 ** 12))
