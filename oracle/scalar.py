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


def minifloat_mx_value(xv: float, E: int, F: int, finite: bool, mode: str):
    """What ``_minifloat_mx/fake.py:11-149`` (encode, then decode) computes for one finite fp32 value, stated on the
    VALUE in exact rationals, with no bit field in sight: |x| = m 2^e; modes other than "rz" first drop what lies below
    2^(e-15); r = the fraction in units of 2^(e-F) rounded in the mode on the magnitude; a fraction that rounds up to
    2^F gives 2^(e+1) when e + bias is even and 2^e when it is odd (into the Inf code at the top of a format that has
    one); e = -bias truncates to the subnormal grid (r = 0: zero; r = 2^F: 2^-bias); below that, and below 2^-126,
    zero; above the top exponent the largest magnitude.  Returns (Fraction | "inf", negative).  The derivation and the
    sweep that holds the vectorised restatement to it are in tests/test_minifloat_mx_value_pins.py."""
    bias = 2 ** (E - 1) - 1
    emax = (2 ** E - 1 if finite else 2 ** E - 2) - bias
    neg = xv < 0
    a = Fraction(abs(xv))
    if a < Fraction(1, 2 ** 126):
        return Fraction(0), neg
    e = 0
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    while Fraction(2) ** e > a:
        e -= 1
    p = lambda k: Fraction(2) ** k
    xt = a if mode == "rz" else (a / p(e - 15)).__floor__() * p(e - 15)
    u = p(e - F)
    q = (xt - p(e)) / u
    fl = q.__floor__()
    if mode == "rn":
        rem = q - fl
        r = fl + (1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1) else 0)
    elif mode == "ru":
        r = fl + (1 if q != fl else 0)
    else:
        r = fl
    if e < -bias:
        return Fraction(0), neg
    if e > emax:
        if emax + bias == 0:
            return (2 ** F - 1) * p(1 - bias - F), neg
        return (2 - p(-F)) * p(emax), neg
    if e == -bias:
        if r == 0:
            return Fraction(0), neg
        if r == 2 ** F:
            return p(-bias), neg
        return ((r + 2 ** F) // 2) * p(1 - bias - F), neg
    if r == 2 ** F:
        if (e + bias) % 2 == 1:
            return p(e), neg
        if not finite and e + bias + 1 == 2 ** E - 1:
            return "inf", neg
        return p(e + 1), neg
    return (2 ** F + r) * u, neg


def minifloat_representable(E: int, F: int, is_finite: bool):
    """all non-negative finite values of the format under the reference's decode"""
    vals = set()
    for c in range(1 << (E + F)):
        v, _ = minifloat_mx_decode(c, E, F, is_finite)
        if not isinstance(v, str):
            vals.add(v)
    return sorted(vals)


# ------------------------------------------------------------------------------------------------
# Explicit-rounding model of the element-wise and block quantizers on 16-bit tensors.
#
# A torch op on a bf16 / fp16 tensor computes in fp32 and stores the result in the tensor dtype.  The functions below
# evaluate the reference's op sequences (block_fp.py:55-80, minifloat.py:46-66, :158-180) in float64, where every
# single op on fp32-representable operands is exact (sums: the smaller addend of a pair more than 29 binades apart
# cannot move the fp32 rounding of the larger), and write every rounding out: ``store(v, fmt)`` = round to fp32, then
# to the dtype, both to nearest even with gradual underflow and overflow to infinity, done with integer scaling, not
# with a library conversion.  The two library-defined pieces are passed in by the caller: log2 as the library rounds
# it in the dtype, and isclose(x, 0).
# ------------------------------------------------------------------------------------------------
import numpy as np

FMT = {  # precision in bits (with the implicit one), exponent of the smallest subnormal step, largest finite value
    "f32": (24, -149, float(np.finfo(np.float32).max)),
    "bf16": (8, -133, 3.3895313892515355e38),
    "f16": (11, -24, 65504.0),
}
EPS_F32 = float(np.float32(1e-9))  # the scalar 1e-9 as the fp32 computation sees it


def round_to(v, fmt: str):
    """round float64 values to the format: nearest even, subnormals, overflow to infinity; NaN and infinity pass"""
    p, qmin, vmax = FMT[fmt]
    v = np.asarray(v, dtype=np.float64)
    out = v.copy()
    fin = np.isfinite(v) & (v != 0)
    m, e = np.frexp(v[fin])                      # |m| in [0.5, 1)
    qe = np.maximum(e - p, qmin)                 # exponent of the rounding step at this magnitude
    r = np.ldexp(np.rint(np.ldexp(v[fin], -qe)), qe)   # rint: nearest even on an exactly scaled value
    r = np.where(np.abs(r) > vmax, np.copysign(np.inf, r), r)
    out[fin] = r
    return out


def store(v, fmt: str):
    """the result of one torch op on a tensor of the format: computed in fp32, stored in the format"""
    return round_to(v, "f32") if fmt == "f32" else round_to(round_to(v, "f32"), fmt)


def _pow2(e, fmt):
    with np.errstate(over="ignore"):
        return store(np.ldexp(1.0, e.astype(np.int64)), fmt)  # 2 ** e on a tensor of integers held in the format


def _select(close, y, x, fmt):
    """(~close) * y + close * x as tensor ops: products with 0.0 / 1.0, then a sum (keeps or loses the sign of zero
    exactly as the float ops do)"""
    with np.errstate(invalid="ignore"):
        return store(store((~close).astype(np.float64) * y, fmt) + store(close.astype(np.float64) * x, fmt), fmt)


def block_fp_model(x, bmax_log2_ceil, close, width: int, exponent_width: int, fmt: str, exponent_bias=None):
    """op-by-op model of block_fp.py:55-80 for elements ``x`` whose block maximum has ceil(log2(max)) =
    ``bmax_log2_ceil`` (as the library rounds it, float64 array of integers or +-inf), ``close`` = isclose(x, 0)"""
    mb = width - 1
    bias = (1 << (exponent_width - 1)) - 1 if exponent_bias is None else exponent_bias
    e_lo, e_hi = float(-bias), float((1 << exponent_width) - 1 - bias)
    m_hi = float(store(np.float64((1 << mb) - 1), fmt))   # a clamp bound is first converted to the dtype
    x = np.asarray(x, dtype=np.float64)
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        sgn = np.sign(store(x + EPS_F32, fmt))
        val = store(np.abs(x) + EPS_F32, fmt)
        e = np.clip(bmax_log2_ceil, e_lo, e_hi)
        p2 = _pow2(e, fmt)
        man = store(val / p2, fmt)
        q = np.clip(np.rint(store(man * float(1 << mb), fmt)), 0.0, m_hi)
        man = store(q / float(1 << mb), fmt)
        y = store(store(sgn * p2, fmt) * man, fmt)
    return _select(close, y, x, fmt)


def block_fp_closed_form(x, e, width: int, fmt: str):
    """the closed form that holds when 2^e, v / 2^e and the final product are exact in the format (widths up to 9 in
    bf16, 12 in fp16, exponents inside the format's normal range): one rounding, that of |x| + 1e-9"""
    mb = width - 1
    x = np.asarray(x, dtype=np.float64)
    v = store(np.abs(x) + EPS_F32, fmt)
    q = np.clip(np.rint(np.ldexp(v, (mb - e).astype(np.int64))), 0.0, float((1 << mb) - 1))
    return np.copysign(np.ldexp(q, (e - mb).astype(np.int64)), x)


def minifloat_model(x, log2_of, close, width: int, exponent_width: int, fmt: str, ieee: bool, exponent_bias=None):
    """op-by-op model of minifloat.py:46-66 (denorm) / :158-180 (ieee).  ``log2_of(v)``: the library's log2 of a
    float64 array of values of the format, evaluated in the format; ``close`` = isclose(|x|, 0)"""
    mb = width - exponent_width - 1
    bias = (1 << (exponent_width - 1)) - 1 if exponent_bias is None else exponent_bias
    e_lo, e_hi = float(-bias), float((1 << exponent_width) - 1 - bias)
    shift = float(1 << mb)
    m_hi = float(store(np.float64((1 << mb) - 1), fmt))
    x = np.asarray(x, dtype=np.float64)
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        sgn = np.sign(store(x + EPS_F32, fmt))
        val = np.abs(x)
        lg = log2_of(store(val + EPS_F32, fmt))
        e = np.clip(np.floor(lg) if ieee else np.ceil(lg), e_lo, e_hi)
        p2 = _pow2(e, fmt)
        man = store(val / p2, fmt)
        if not ieee:
            q = np.clip(np.rint(store(man * shift, fmt)), 0.0, m_hi)
            man = store(q / shift, fmt)
        else:
            normal = ~(e == -float(bias))     # isclose(e, -bias) on integers held exactly in the format
            nf = normal.astype(np.float64)
            qn = np.clip(np.rint(store(store(man * shift, fmt) - shift, fmt)), 0.0, m_hi)
            qs = np.clip(np.rint(store(store(man * shift, fmt) / 2.0, fmt)), 0.0, m_hi)
            q = store(store(nf * qn, fmt) + store((1.0 - nf) * qs, fmt), fmt)
            mn = store(1.0 + store(q / shift, fmt), fmt)
            ms = store(store(q / shift, fmt) * 2.0, fmt)
            man = store(store(nf * mn, fmt) + store((1.0 - nf) * ms, fmt), fmt)
        y = store(store(sgn * p2, fmt) * man, fmt)
    return _select(close, y, x, fmt)
