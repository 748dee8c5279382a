"""Value-domain pins for the `_minifloat_mx` cast (no GPU, no bit fields).

``oracle.minifloat_quantizer_sim`` restates `_minifloat_mx/fake.py:11-149` as operations on bit fields.  This file
states what that text computes as a function of the input VALUE, in exact arithmetic, and compares the two over every
16-bit high-half fp32 pattern, the same patterns with non-zero low halves, and a dense grid of rounding ties and
near-ties, for every legal MXFP element format (mxfp/meta.py:41), both ``is_finite`` settings and all four rounding
modes.  The arithmetic is float64 on fp32 inputs scaled by powers of two, floored or rounded to integers below 2^53:
every operation is exact (a sample is re-done in ``fractions.Fraction`` to hold that claim).

What the text fixes, as values (|x| = m * 2^e, 1 <= m < 2; bias = 2^(E-1) - 1; emax = the largest exponent field
minus bias; u = 2^(e-F) the spacing of the format in the binade of x):

 (o)   modes other than "rz" first drop the low 8 mantissa bits of x (fake.py:59, ``>> 8``): x' = the multiple of
       2^(e-15) next to x towards zero; "rz" keeps x (fake.py:57).  r = round((|x'| - 2^e) / u) in the mode, on the
       magnitude (fake.py:60-69): "ru" is away from zero, "rd" and "rz" towards zero, "rn" ties-to-even.
 (i)   carry: r = 2^F.  The fraction is OR-ed into the exponent field (fake.py:89), so the result is 2^(e+1) when
       the field e + bias is even and stays 2^e when it is odd.  In a format with Inf/NaN codes an even field at the
       top of the range carries into the Inf code.
 (ii)  e = -bias (exponent field 0, fake.py:71-72): r = 0 gives zero; 0 < r < 2^F gives
       floor((r + 2^F) / 2) * 2^(1-bias-F), a truncation; r = 2^F gives 2^-bias (the OR again: 2^F | 2^F = 2^F).
 (iii) e < -bias, or |x| below 2^-126 (fake.py:37, 49, 75-76): zero, with the sign of x (x = -0.0 gives +0.0, since
       the sign is ``x < 0``, fake.py:35).
 (iv)  e > emax (fake.py:78-79): the largest magnitude (2 - 2^-F) * 2^emax; with ``is_finite`` emax = 2^E - 1 - bias,
       else 2^E - 2 - bias.
 (v)   elsewhere (2^F + r) * u: the representable value nearest to x' in the mode.
 (vi)  ``is_finite=False``: +-Inf encodes with exponent field 2^E - 2 and fraction 0 (fake.py:82-87), which decodes
       as the ordinary value 2^emax; NaN with that field and fraction 2^F - 1, the largest magnitude, sign +.
       Inf/NaN into an all-finite format goes through ``frexp`` of a non-finite value: unspecified, not swept.
 (vii) E = 1 with ``is_finite=False`` is degenerate: the largest exponent field is 0, so the codes of (iv) and (vi)
       have exponent field 0 and decode as the format's subnormals (fake.py:127-137): overflow and NaN give
       (2^F - 1) * 2^(1-bias-F), Inf gives zero.

Mutations of the closed form (ADD for the OR, a rounded instead of truncated exponent-field-0 region, rounding before
the 8-bit truncation, gradual underflow below 2^-bias, a "ru" towards +Inf, the largest exponent of the other
``is_finite`` setting) are each shown to disagree with the oracle on the swept set, so the sweep does reach every region.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle as O
from oracle.scalar import minifloat_mx_value as closed_form_fraction

FORMATS = [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2)]  # mxfp/meta.py:41
MODES = ["rn", "ru", "rd", "rz"]


def closed_form(x: np.ndarray, E: int, F: int, finite: bool, mode: str, mutant: str = "") -> np.ndarray:
    """float64 in (fp32-representable values), float64 out; NaN inputs only with ``finite=False``"""
    bias = 2 ** (E - 1) - 1
    emax = (2 ** E - 1 if finite else 2 ** E - 2) - bias
    if mutant == "other_emax":
        emax = (2 ** E - 2 if finite else 2 ** E - 1) - bias
    neg = x < 0
    a = np.abs(x)
    nan_in = np.isnan(a)
    inf_in = np.isinf(a)
    a = np.where(nan_in | inf_in, 1.0, a)
    flushed = a < 2.0 ** -126
    a = np.where(flushed, 1.0, a)  # placeholder value; overwritten below
    _, ex = np.frexp(a)
    e = ex.astype(np.int64) - 1
    two_e = np.ldexp(1.0, e)
    if mode == "rz" or mutant == "round_before_truncation":
        xt = a
    else:
        g = np.ldexp(1.0, e - 15)
        xt = np.floor(a / g) * g
    u = np.ldexp(1.0, e - F)
    q = (xt - two_e) / u
    if mode == "rn":
        r = np.rint(q)  # ties to even
    elif mode == "ru":
        r = np.ceil(q)
        if mutant == "ru_towards_plus_inf":
            r = np.where(neg, np.floor(q), r)
    else:
        r = np.floor(q)
    full = float(2 ** F)
    carry = r == full
    field = e + bias
    val = (full + r) * u  # (v)
    if mutant == "add_for_or":
        up = np.ones_like(carry)
    else:
        up = field % 2 == 0
    top = np.ldexp(1.0, e + 1)
    if not finite:
        top = np.where(field + 1 == 2 ** E - 1, np.inf, top)
    val = np.where(carry, np.where(up, top, two_e), val)  # (i)
    # (ii)
    unit = 2.0 ** (1 - bias - F)
    if mutant == "rounded_subnormals":
        sub = np.rint((r + full) / 2) * unit
    else:
        sub = np.floor((r + full) / 2) * unit
    sub = np.where(carry, 2.0 ** -bias if mutant != "add_for_or" else 2.0 ** (1 - bias), sub)
    sub = np.where(r == 0, 0.0, sub)
    val = np.where(field == 0, sub, val)
    # (iii), (iv)
    if mutant == "gradual_underflow":
        below = np.rint(xt / unit) * unit
        val = np.where(e < -bias, below, val)
    else:
        val = np.where(e < -bias, 0.0, val)
    largest = (2.0 - 2.0 ** -F) * 2.0 ** emax
    inf_value = 2.0 ** emax
    if emax + bias == 0:  # (vii)
        largest, inf_value = (2 ** F - 1) * unit, 0.0
    val = np.where(e > emax, largest, val)
    val = np.where(flushed, 0.0, val)
    if not finite:  # (vi)
        val = np.where(inf_in, inf_value, val)
        val = np.where(nan_in, largest, val)
    return np.where(neg, -val, val)


def swept_bits(E: int, F: int) -> np.ndarray:
    """every high-half pattern, the same with random and extreme low halves, and for every fp32 exponent around the
    format's range every grid point of the binade with offsets (in units of the 15-bit truncated mantissa) around the
    rounding ties and the binade's end, each with low 8 bits 0x00, 0x01 and 0xFF"""
    rng = np.random.default_rng(100 * E + F)
    hi = np.arange(65536, dtype=np.uint32) << 16
    parts = [hi, hi | rng.integers(0, 1 << 16, 65536).astype(np.uint32), hi | np.uint32(0xFFFF), hi | np.uint32(0x00FF),
             hi | np.uint32(0x8000), hi | np.uint32(0x7FFF), hi | np.uint32(0x80FF)]
    bias = 2 ** (E - 1) - 1
    exps = np.arange(-bias - 3, 2 ** E - bias + 3)
    exps = np.concatenate([exps, [-126, -125, -60, 60, 126, 127]])
    step = 1 << (15 - F)  # one grid step in 15-bit mantissa units
    m15 = []
    for r in range(2 ** F):
        for off in (0, 1, step // 2 - 1, step // 2, step // 2 + 1, step - 1):
            m15.append(r * step + off)
    m15 = np.unique(np.array(m15, dtype=np.uint32))
    grid = []
    for low in (0x00, 0x01, 0xFF):
        man = (m15 << 8) | np.uint32(low)
        for ex in exps:
            for s in (0, 1):
                grid.append((np.uint32(s) << 31) | (np.uint32(ex + 127) << 23) | man)
    parts.append(np.concatenate(grid))
    # fp32 subnormals, zeros, infinities
    parts.append(np.array([0, 0x80000000, 1, 0x80000001, 0x007FFFFF, 0x807FFFFF, 0x00800000, 0x80800000,
                           0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000, 0x7FC00000], dtype=np.uint32))
    return np.unique(np.concatenate(parts))


def oracle_values(bits: np.ndarray, E, F, finite, mode) -> np.ndarray:
    x = torch.from_numpy(bits.view(np.int32).copy()).view(torch.float32)
    return O.minifloat_quantizer_sim(x, E, F, finite, mode).numpy()


def select_inputs(bits: np.ndarray, finite: bool) -> np.ndarray:
    if finite:  # Inf/NaN into a format without them: unspecified
        return bits[(bits & np.uint32(0x7F800000)) != np.uint32(0x7F800000)]
    return bits


def same_bits(got32: np.ndarray, want64: np.ndarray) -> np.ndarray:
    want32 = want64.astype(np.float32)
    assert np.array_equal(want32.astype(np.float64), want64, equal_nan=True), "closed form left the fp32 grid"
    return (got32.view(np.uint32) == want32.view(np.uint32)) | (np.isnan(got32) & np.isnan(want32))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("finite", [True, False])
@pytest.mark.parametrize("E,F", FORMATS)
def test_cast_equals_the_value_domain_closed_form(E, F, finite, mode):
    bits = select_inputs(swept_bits(E, F), finite)
    got = oracle_values(bits, E, F, finite, mode)
    with np.errstate(invalid="ignore"):  # signalling NaN patterns among the inputs
        want = closed_form(bits.view(np.float32).astype(np.float64), E, F, finite, mode)
    ok = same_bits(got, want)
    if not ok.all():
        i = int(np.flatnonzero(~ok)[0])
        raise AssertionError(f"{(~ok).sum()} of {ok.size} differ; first: bits 0x{int(bits[i]):08x} "
                             f"x={bits.view(np.float32)[i]!r} oracle={got[i]!r} closed form={want[i]!r}")


MUTANTS = ["add_for_or", "rounded_subnormals", "round_before_truncation", "gradual_underflow",
           "ru_towards_plus_inf", "other_emax"]


@pytest.mark.parametrize("mutant", MUTANTS)
@pytest.mark.parametrize("E,F", FORMATS)
def test_the_sweep_tells_plausible_misreadings_apart(E, F, mutant):
    """each misreading of the source must disagree with the oracle somewhere on the swept inputs"""
    mode = "ru" if mutant == "ru_towards_plus_inf" else "rn"
    bits = select_inputs(swept_bits(E, F), True)
    got = oracle_values(bits, E, F, True, mode)
    x = bits.view(np.float32).astype(np.float64)
    wrong = closed_form(x, E, F, True, mode, mutant).astype(np.float32)
    right = closed_form(x, E, F, True, mode).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), right.view(np.uint32))
    differ = int((wrong.view(np.uint32) != got.view(np.uint32)).sum())
    assert differ > 0, f"mutant {mutant} is not told apart for e{E}m{F}"


@pytest.mark.parametrize("E,F", FORMATS)
def test_float64_closed_form_is_exact(E, F):
    """the float64 statement against the same statement in rationals, on a sample across all regions"""
    bits = select_inputs(swept_bits(E, F), True)
    rng = np.random.default_rng(7)
    bias = 2 ** (E - 1) - 1
    ex = ((bits >> 23) & 0xFF).astype(np.int64) - 127
    near = (ex >= -bias - 2) & (ex <= 2 ** E - bias + 1)
    pick = np.concatenate([rng.choice(np.flatnonzero(near), 1500, replace=False),
                           rng.choice(np.flatnonzero(~near), 300, replace=False)])
    xs = bits[pick].view(np.float32).astype(np.float64)
    for finite in (True, False):
        for mode in MODES:
            vals = closed_form(xs, E, F, finite, mode)
            for xv, v in zip(xs.tolist(), vals.tolist()):
                want, neg = closed_form_fraction(xv, E, F, finite, mode)
                if want == "inf":
                    assert v == (-np.inf if neg else np.inf)
                else:
                    assert Fraction(v) == (-want if neg else want), (xv, v, want)
                    assert v != 0 or (np.signbit(v) == neg)


def test_known_values_follow_from_the_closed_form():
    """hand-evaluated instances of (i)-(iv), as numbers a reader can redo on paper"""
    q = lambda v, E, F, fin=True, rm="rn": float(O.minifloat_quantizer_sim(torch.tensor([v], dtype=torch.float32), E, F, fin, rm))
    # (i) e4m3, bias 7: 500 = 1.953 * 2^8, field 15 (odd): r = rne(0.953 * 8) = 8 = 2^F -> stays 2^8
    assert q(500.0, 4, 3) == 256.0
    # (i) e4m3: 250 = 1.953 * 2^7, field 14 (even) -> 2^8
    assert q(250.0, 4, 3) == 256.0
    # (i) with Inf/NaN codes the largest field is 14 (even): 250 is in the top binade and carries into the Inf code
    assert q(250.0, 4, 3, False) == float("inf")
    # (ii) e4m3, e = -7: x = 1.5 * 2^-7: r = 4 -> floor((4 + 8) / 2) = 6 units of 2^-9 = 1.5 * 2^-7 (exact here)
    assert q(1.5 * 2.0 ** -7, 4, 3) == 6 * 2.0 ** -9
    # (ii) 1.625 * 2^-7: r = 5 -> floor(13 / 2) = 6 units: truncated, the nearest would be 6.5 -> 6 (tie) - take 1.875:
    # r = 7 -> floor(15 / 2) = 7 units = 1.75 * 2^-7, while the nearest multiple of 2^-9 to 7.5 units is 8 (ties-even)
    assert q(1.875 * 2.0 ** -7, 4, 3) == 7 * 2.0 ** -9
    # (ii) r = 0: 2^-7 itself is flushed to zero; r = 2^F: 1.97 * 2^-7 gives 2^-7
    assert q(2.0 ** -7, 4, 3) == 0.0
    assert q(1.97 * 2.0 ** -7, 4, 3) == 2.0 ** -7
    # (iii) / (iv)
    assert q(2.0 ** -8 * 1.9, 4, 3) == 0.0 and q(1e9, 4, 3) == 480.0 and q(1e9, 4, 3, False) == 240.0
    # (o) 1 + 2^-4 + 2^-23: after the 8-bit truncation an exact tie (r = 0.5 -> 0, even); without it, above the tie
    assert q(1.0 + 2.0 ** -4 + 2.0 ** -23, 4, 3) == 1.0
    assert q(1.0 + 2.0 ** -4 + 2.0 ** -15, 4, 3) == 1.125
