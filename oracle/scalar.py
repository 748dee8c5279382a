"""Independent scalar restatements (pure Python integers / fractions) used to pin ``oracle.quantizers``.

TEST INFRASTRUCTURE.  Nothing here shares code with the vectorised torch restatement: these routines work
on one value at a time with exact rational arithmetic, so a transposed operand, a wrong rounding rule or a
missed clamp in either restatement shows up as a disagreement.  Where the reference's behaviour is *not* the
textbook one (documented quirks of ``_minifloat_mx/fake.py``), the quirk is stated as such and implemented
here from the source text a second time; outside those regions the result is additionally checked against
"nearest representable value" brute force in the tests.
"""
from __future__ import annotations

import struct
from fractions import Fraction


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bits_f32(b: int) -> float:
    return struct.unpack("<f", struct.pack("<I", b & 0xFFFFFFFF))[0]


def rne(fr: Fraction) -> int:
    """round half to even on an exact rational"""
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        return fl + 1
    return fl


# ------------------------------------------------------------------------------------------------
# fixed point: clamp(rne(x * 2^f), lo, hi) / 2^f   (integer.py:10-46)
# ------------------------------------------------------------------------------------------------
def integer_quantize(x: float, width: int, frac_width: int, is_signed: bool = True, floor: bool = False) -> Fraction:
    v = Fraction(x) * (Fraction(2) ** frac_width)
    q = (v.numerator // v.denominator) if floor else rne(v)
    lo, hi = (-(1 << (width - 1)), (1 << (width - 1)) - 1) if is_signed else (0, (1 << width) - 1)
    q = min(max(q, lo), hi)
    return Fraction(q) / (Fraction(2) ** frac_width)


# ------------------------------------------------------------------------------------------------
# MXINT block given its exponent k (the exponent itself comes from the library's log2: mxint/fake.py:45)
# ------------------------------------------------------------------------------------------------
def mxint_block(xs, k: int, element_bits: int, scale_bits: int = 8):
    """exact dequantized values of one block, as Fractions (mxint/fake.py:47-54, 75-80)"""
    b = element_bits
    bias = (1 << (scale_bits - 1)) - 1
    kc = min(max(k + bias, 0), (1 << scale_bits) - 1) - bias
    out = []
    for x in xs:
        m = rne(Fraction(x) / (Fraction(2) ** k) * (1 << (b - 1)))
        m = min(max(m, -(1 << (b - 1))), (1 << (b - 1)) - 1)
        out.append(Fraction(m, 1 << (b - 1)) * (Fraction(2) ** kc))
    return out


# ------------------------------------------------------------------------------------------------
# block floating point given the block exponent e (block_fp.py:55-80), exact in fp32
# ------------------------------------------------------------------------------------------------
def block_fp_element_f32(x: float, e: int, width: int) -> Fraction:
    """value of one non-'close' element in fp32: sign(x) * 2^e * clamp(rne((|x|+1e-9f)/2^e * 2^mb), 0, 2^mb-1) / 2^mb,
    where |x| + 1e-9f is an fp32 addition (performed by the caller-independent struct round trip)."""
    mb = width - 1
    v = bits_f32(f32_bits(abs(x) + bits_f32(f32_bits(1e-9))))  # fp32 sum, rounded once
    q = rne(Fraction(v) / (Fraction(2) ** e) * (1 << mb))
    q = min(max(q, 0), (1 << mb) - 1)
    y = Fraction(q, 1 << mb) * (Fraction(2) ** e)
    return -y if x < 0 else y


# ------------------------------------------------------------------------------------------------
# _minifloat_mx encode / decode on one fp32 bit pattern (fake.py:11-149)
# ------------------------------------------------------------------------------------------------
def minifloat_mx_encode(xbits: int, E: int, F: int, is_finite: bool, round_mode: str) -> int:
    bias = (1 << (E - 1)) - 1
    e_hi = (1 << E) - 1 if is_finite else (1 << E) - 2
    sign = 1 if (xbits >> 31) and (xbits & 0x7FFFFFFF) != 0 and (xbits & 0x7FFFFFFF) <= 0x7F800000 else 0  # x < 0
    ab = xbits & 0x7FFFFFFF
    expf = ab >> 23
    man = ab & 0x7FFFFF
    is_inf = ab == 0x7F800000
    is_nan = ab > 0x7F800000
    ftz = expf == 0
    if ftz:
        e, man = -1, 0  # frexp(0) = (0, 0): exponent 0 - 1
    elif is_inf or is_nan:
        e = -1  # the library's frexp returns exponent 0 for non-finite input
    else:
        e = expf - 127
    under = e < -bias
    over = e > e_hi - bias
    ye = e + bias
    if round_mode == "rz":
        yf = man >> (23 - F)
    else:
        m15 = man >> 8  # the low 8 mantissa bits are dropped before rounding (fake.py:54)
        v = Fraction(m15, 1 << (15 - F))
        if round_mode == "rn":
            yf = rne(v)
        elif round_mode == "ru":
            yf = -((-v.numerator) // v.denominator)
        elif round_mode == "rd":
            yf = v.numerator // v.denominator
        else:
            raise ValueError(round_mode)
    if ye == 0 and yf != 0:
        yf = (yf | (1 << F)) >> 1
    if under:
        yf, ye = 0, 0
    if over:
        yf, ye = (1 << F) - 1, e_hi
    if ftz:
        yf, ye = 0, 0
    if not is_finite:
        if is_inf:
            yf, ye = 0, e_hi
        if is_nan:
            yf, ye = (1 << F) - 1, e_hi
    y = (ye << F) | yf  # a fraction of 2^F collides with the exponent field: OR, not ADD (fake.py:89)
    if sign:
        y += 1 << (E + F)
    return y & 0xFFFF


def minifloat_mx_decode(code: int, E: int, F: int, is_finite: bool):
    """exact value as a Fraction, or the strings 'inf'/'-inf'/'nan'; the sign of zero as (Fraction(0), sign)"""
    bias = (1 << (E - 1)) - 1
    sgn = (code >> (E + F)) & 1
    c = code & 0x7FFF
    xe = (c >> F) & ((1 << E) - 1)
    xf = c & ((1 << F) - 1)
    if not is_finite and xe == (1 << E) - 1:
        return ("nan" if xf else ("-inf" if sgn else "inf")), sgn
    if xe == 0:
        v = Fraction(xf, 1 << F) * Fraction(2) ** (1 - bias)
    else:
        v = (1 + Fraction(xf, 1 << F)) * Fraction(2) ** (xe - bias)
    return (-v if sgn else v), sgn


def minifloat_representable(E: int, F: int, is_finite: bool):
    """all non-negative finite values of the format under the reference's decode"""
    vals = set()
    for c in range(1 << (E + F)):
        v, _ = minifloat_mx_decode(c, E, F, is_finite)
        if not isinstance(v, str):
            vals.add(v)
    return sorted(vals)
