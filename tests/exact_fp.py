"""Exact arithmetic for pinning the quantizer's rounding points (test infrastructure).

Two independent restatements of "round to nearest, ties to even, into a binary floating-point format"
that share no code with numpy's float16 arithmetic or with the oracle:

* `rne` on `fractions.Fraction`: the textbook definition, one value at a time;
* `quantize_codes_int`: the whole quantizer of group_quantization.py:250-287 in numpy int64
  (significand / exponent pairs, long division with remainder), fast enough for millions of values.

A format is (p, emin): p significand bits including the hidden one, emin the exponent of the smallest
normal number.  binary16 = (11, -14), bfloat16 = (8, -126), binary32 = (24, -126).
"""

from __future__ import annotations

from fractions import Fraction

import numpy as np

FORMATS = {"float16": (11, -14), "bfloat16": (8, -126), "float32": (24, -126)}
_EMAX = {"float16": 15, "bfloat16": 127, "float32": 127}
INF = Fraction(10) ** 60  # stands for +infinity; nothing finite here comes near it


def _floor_log2(a: Fraction) -> int:
    """floor(log2(a)) for a > 0, exactly."""
    e = a.numerator.bit_length() - a.denominator.bit_length()
    # 2^e <= a < 2^(e+1) may be off by one: fix up with exact comparisons
    if Fraction(2) ** e > a:
        e -= 1
    elif Fraction(2) ** (e + 1) <= a:
        e += 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    return e


def rne(x: Fraction, fmt: str) -> Fraction:
    """x rounded to the nearest value of the format, ties to the even significand; subnormals are
    multiples of 2^(emin-p+1); magnitudes at or beyond the overflow threshold become +-INF."""
    p, emin = FORMATS[fmt]
    if x == 0:
        return Fraction(0)
    if abs(x) >= INF:
        return INF if x > 0 else -INF
    sign = 1 if x > 0 else -1
    a = abs(x)
    e = max(_floor_log2(a), emin)
    quantum = Fraction(2) ** (e - (p - 1))
    n = a / quantum
    f = n.numerator // n.denominator
    rem = n - f
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and f % 2 == 1):
        f += 1
    r = f * quantum
    if r >= Fraction(2) ** (_EMAX[fmt] + 1):
        return sign * INF
    return sign * r


def _round_half(t: Fraction, mode: str) -> Fraction:
    if abs(t) >= INF:
        return t
    fl = t.numerator // t.denominator
    frac = t - fl
    if frac == Fraction(1, 2):
        if mode == "half_away":
            return Fraction(fl + 1 if t > 0 else fl)
        return Fraction(fl if fl % 2 == 0 else fl + 1)
    return Fraction(fl + 1 if frac > Fraction(1, 2) else fl)


def quantize_group_fraction(w: list, m: int, fmt: str, mode: str = "half_away", roundings: int = 2):
    """One group of group_quantization.py:250-287 in exact rationals.

    w: the group's values as Fractions (already values of the format).  roundings = 2 is the
    reference's order (quotient rounded to the format, then the sum with m rounded again);
    roundings = 1 rounds only once, after the add, which is the mistake the two-rounding tests must
    catch.  Returns (codes, scale as Fraction)."""
    max_abs = max(abs(v) for v in w)
    scale = rne(max_abs / m, fmt)
    codes = []
    for v in w:
        if scale == 0:
            # IEEE: 0/0 is NaN and the compare-select maximum with 0 yields 0; x/0 is +-inf
            t = None if v == 0 else (INF if v > 0 else -INF)
        elif roundings == 2:
            t = rne(rne(v / scale, fmt) + m, fmt)
        else:
            t = rne(v / scale + m, fmt)
        if t is None:
            codes.append(0)
            continue
        r = _round_half(t, mode)
        r = r if r > 0 else Fraction(0)
        r = r if r < 2 * m else Fraction(2 * m)
        codes.append(int(r))
    return codes, scale


def to_fraction(a: np.ndarray) -> list:
    """Finite float16 / float32 values as exact Fractions (a float's value is a dyadic rational)."""
    return [Fraction(float(v)) for v in np.asarray(a).ravel()]


# --------------------------------------------------------------------------- int64, vectorised


def _decompose(bits: np.ndarray, fmt: str):
    """Raw encodings -> (sign, significand, exponent) with value = sign * significand * 2^exponent.
    bits: uint16 encodings for float16, the upper 16 bits of a float32 for bfloat16."""
    b = bits.astype(np.int64)
    if fmt == "float16":
        ebits, fbits, bias = 5, 10, 15
    elif fmt == "bfloat16":
        ebits, fbits, bias = 8, 7, 127
    else:
        raise ValueError(fmt)
    sign = np.where((b >> (ebits + fbits)) & 1, -1, 1).astype(np.int64)
    e = (b >> fbits) & ((1 << ebits) - 1)
    frac = b & ((1 << fbits) - 1)
    assert (e != (1 << ebits) - 1).all(), "finite values only"
    sig = np.where(e > 0, frac + (1 << fbits), frac)
    exp = np.maximum(e, 1) - bias - fbits
    return sign, sig, exp


def _rne_int(q: np.ndarray, sticky: np.ndarray, base: np.ndarray, fmt: str):
    """Round (q + sticky_fraction) * 2^base, 0 <= q < 2^48 int64, to the format (sticky_fraction is
    some value in (0, 1) where `sticky` is set, else 0).  Returns (f, eq) with the rounded magnitude =
    f * 2^eq."""
    p, emin = FORMATS[fmt]
    assert (q >= 0).all() and (q < (np.int64(1) << 48)).all()
    q = q << 14  # room below the last kept bit, so that a short q is never shifted left here
    base = base - 14
    length = np.zeros_like(q)
    nz = q > 0
    # bit length by float64 log2 is unsafe near powers of two: count with shifts instead
    tmp = q.copy()
    for s in (32, 16, 8, 4, 2, 1):
        big = tmp >= (np.int64(1) << s)
        length = np.where(big, length + s, length)
        tmp = np.where(big, tmp >> s, tmp)
    length = np.where(nz, length + 1, 0)
    e = length - 1 + base
    eq = np.maximum(e, emin) - (p - 1)
    sh = np.clip(eq - base, 1, 62)
    f = q >> sh
    rem = q & ((np.int64(1) << sh) - 1)
    half = np.int64(1) << (sh - 1)
    up = (rem > half) | ((rem == half) & sticky) | ((rem == half) & ~sticky & ((f & 1) == 1))
    f = np.where(up, f + 1, f)
    return np.where(nz, f, 0), eq


def quantize_codes_int(w_bits: np.ndarray, group: int, m: int, fmt: str, mode: str = "half_away",
                       roundings: int = 2) -> np.ndarray:
    """Codes of group_quantization.py:274-287 for [rows, K] raw encodings (K a multiple of the group
    size, no group with a zero or subnormal-quotient scale: callers pass ordinary weight data), by long
    division in int64.  roundings = 1: the quotient is kept as quotient and remainder and rounded only after the add."""
    p, emin = FORMATS[fmt]
    rows, k = w_bits.shape
    assert k % group == 0
    sign, sig, exp = _decompose(w_bits, fmt)
    # max |w| per group: compare (exp, sig) after aligning to the group's smallest exponent
    val_key = sig.astype(np.float64) * np.exp2(exp.astype(np.float64))  # exact: 11 bits x power of two
    g_key = val_key.reshape(rows, k // group, group)
    arg = g_key.argmax(-1)
    take = lambda a: np.take_along_axis(a.reshape(rows, k // group, group), arg[..., None], -1)[..., 0]
    msig, mexp = take(sig), take(exp)
    assert (msig > 0).all(), "all-zero groups are not handled here"
    # scale = rne(max_abs / m)
    num = msig << 24
    sq, sr = num // m, num % m
    s_f, s_eq = _rne_int(sq, sr != 0, mexp - 24, fmt)
    assert (s_f > 0).all()
    s_f = np.repeat(s_f, group, axis=-1)
    s_eq = np.repeat(s_eq, group, axis=-1)
    # quotient w / scale
    shift = 24 if roundings == 2 else 30
    num = sig << shift
    q, r = num // s_f, num % s_f
    base = exp - s_eq - shift
    if roundings == 2:
        t_f, t_eq = _rne_int(q, r != 0, base, fmt)
        sticky = np.zeros_like(q, dtype=bool)
    else:
        # keep the exponent within reach of the shift below: bits under 2^-40 only matter as "not zero"
        drop = np.clip(-40 - base, 0, 62)
        t_f, t_eq, sticky = q >> drop, base + drop, (r != 0) | ((q & ((np.int64(1) << drop) - 1)) != 0)
    # t + m on the common exponent (t_eq < 0 for every quotient of magnitude below 2^(p-1)); a zero
    # quotient carries no exponent of its own
    # quotient carries no exponent of its own, and one below 2^-30 cannot move the rounding of m + t (m is a
    # value of the format and its neighbours are at least 2^-22 away), so it is dropped before the shift
    tiny = t_f.astype(np.float64) * np.exp2(t_eq.astype(np.float64)) < 2.0**-30
    sticky = sticky & ~tiny
    t_f = np.where(tiny, 0, t_f)
    t_eq = np.where(tiny, 0, t_eq)
    assert (t_eq <= 0).all() and (t_eq >= -60).all()
    total = sign * t_f + (np.int64(m) << (-t_eq))
    # for negative quotients the sticky remainder pulls towards zero, i.e. the exact sum is total - fraction
    neg_sticky = sticky & (sign < 0)
    total = np.where(neg_sticky, total - 1, total)  # exact sum = total + fraction in (0, 1)
    # a scale that was rounded down makes -max|w| / scale + m slightly negative: every negative sum, rounded
    # either way, ends at or below zero and the maximum with 0 makes it code 0
    negative = total < 0
    total = np.where(negative, 0, total)
    u_f, u_eq = _rne_int(total, sticky & ~negative, t_eq, fmt)
    # integer rounding of u = u_f * 2^u_eq
    assert (u_eq <= 0).all()
    one = np.int64(1) << (-u_eq)
    fl = u_f >> (-u_eq)
    rem = u_f & (one - 1)
    half = one >> 1
    if mode == "half_away":
        up = (u_eq < 0) & (rem >= half)
    else:
        up = (u_eq < 0) & ((rem > half) | ((rem == half) & ((fl & 1) == 1)))
    code = np.where(negative, 0, np.where(up, fl + 1, fl))
    return np.clip(code, 0, 2 * m).astype(np.uint32)
