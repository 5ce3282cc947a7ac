"""Exact rational arithmetic with explicit IEEE roundings, used to pin the CPU checker.

Nothing here shares code with the checker: values are ``fractions.Fraction`` and every rounding to
binary32 / bfloat16 is done by integer arithmetic (round to nearest, ties to even, gradual underflow).
"""
from __future__ import annotations

import struct
from fractions import Fraction


def f32_bits_to_fraction(u: int) -> Fraction:
    sign = -1 if (u >> 31) else 1
    e = (u >> 23) & 0xFF
    m = u & 0x7FFFFF
    assert e != 255, "finite values only"
    if e == 0:
        return sign * Fraction(m, 1 << 149)
    return sign * Fraction((1 << 23) | m) * Fraction(2) ** (e - 150)


def float_to_fraction(x: float) -> Fraction:
    """x must already be a binary32 value held in a Python float."""
    return f32_bits_to_fraction(struct.unpack("<I", struct.pack("<f", x))[0])


def _round_half_even(fr: Fraction) -> int:
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        return fl + 1
    return fl


def rn(fr: Fraction, mant_bits: int, emin: int) -> Fraction:
    """Round to nearest-even onto a binary format with `mant_bits` significand bits (incl. hidden bit)
    and minimum normal exponent `emin`; no overflow handling (callers stay in range)."""
    if fr == 0:
        return Fraction(0)
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    e = max(e, emin)
    quantum = Fraction(2) ** (e - (mant_bits - 1))
    n = _round_half_even(a / quantum)
    r = n * quantum
    return r if fr > 0 else -r


def rn32(fr: Fraction) -> Fraction:
    return rn(fr, 24, -126)


def rn_bf16(fr: Fraction) -> Fraction:
    return rn(fr, 8, -126)


def rn_f16(fr: Fraction) -> Fraction:
    return rn(fr, 11, -14)


def quantize_block_exact(xs):
    """xs: list of Fractions (exactly the input values).  Returns (scale Fraction, list of int codes)
    following  code = rint_even( RN32( 127 * RN32( x / absmax ) ) )."""
    s = max((abs(v) for v in xs), default=Fraction(0))
    if s == 0:
        return s, [0] * len(xs)
    codes = []
    for v in xs:
        quot = rn32(v / s)
        t = rn32(127 * quot)
        codes.append(_round_half_even(t))
    return s, codes


def dequantize_exact(s: Fraction, code: int, out: str = "bf16") -> Fraction:
    inv127 = float_to_fraction(struct.unpack("<f", struct.pack("<f", 1.0 / 127.0))[0])
    v = rn32(rn32(s * code) * inv127)
    return {"bf16": rn_bf16, "f32": lambda z: z, "f16": rn_f16}[out](v)
