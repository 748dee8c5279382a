#!/usr/bin/env python3
"""Writes tests/golden/known_answers.json: small known-answer vectors for the quantize-dequantize functions.

The expected outputs do NOT come from the reference implementation (running it to write vectors was not possible
in the build environment) and NOT from the vectorised oracle: they are computed here one value at a time with exact
rational arithmetic from the format definitions (``oracle/scalar.py``), with block exponents obtained by exact
integer comparison.  Inputs are drawn so that no block maximum lies within 2^-10 (relative) of a power of two,
which keeps the expected values independent of how a math library rounds log2.  The file holds fp32 bit patterns.

    python tests/golden/make_known_answers.py
"""
import json
import os
import random
import struct
import sys
from fractions import Fraction

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import scalar as S  # noqa: E402


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def frac_bits(fr, negative_zero=False):
    """fp32 bit pattern of an exactly representable rational"""
    v = float(fr)
    assert Fraction(v) == fr and f32(v) == v, fr
    b = bits(v)
    return b | 0x80000000 if (fr == 0 and negative_zero) else b


def exact_floor_log2(v):
    fr = Fraction(v)
    k = 0
    while Fraction(2) ** (k + 1) <= fr:
        k += 1
    while Fraction(2) ** k > fr:
        k -= 1
    return k


def safe_block(rng, n, scale):
    """n fp32 values whose largest magnitude is comfortably inside a binade"""
    while True:
        xs = [f32(rng.gauss(0.0, 1.0) * scale) for _ in range(n)]
        m = max(abs(x) for x in xs)
        k = exact_floor_log2(m)
        r = m / 2.0 ** k
        if 1.001 < r < 1.999:
            return xs


def main():
    rng = random.Random(20240917)
    out = {"integer": [], "mxint": [], "block_fp": [], "mxfp": []}
    for width, frac in ((8, 4), (4, 1), (12, 10)):
        xs = [f32(rng.gauss(0.0, 3.0)) for _ in range(48)] + [0.0, -0.0, 0.03125, -0.03125, 1e-6, -1e-6, 200.0, -200.0]
        for floor in (False, True):
            ys = []
            for x in xs:
                q = S.integer_quantize(x, width, frac, True, floor)
                # round(-0.3) is -0.0: the sign of a zero result follows the input
                ys.append(frac_bits(q, negative_zero=(q == 0 and (x < 0 or bits(x) >> 31))))
            out["integer"].append({"width": width, "frac_width": frac, "floor": floor,
                                   "x": [bits(x) for x in xs], "y": ys})
    for ebits in (8, 4):
        for scale in (1.0, 0.02, 37.0):
            xs = safe_block(rng, 32, scale)
            m = max(abs(x) for x in xs)
            k = exact_floor_log2(m) + 1  # ceil(log2 m) for m not a power of two
            ys = S.mxint_block(xs, k, ebits, 8)
            out["mxint"].append({"block_size": 32, "element_bits": ebits, "x": [bits(x) for x in xs],
                                 "y": [frac_bits(y, negative_zero=(y == 0 and x < 0)) for x, y in zip(xs, ys)]})
    for width in (8, 6):
        for scale in (1.0, 50.0):
            xs = safe_block(rng, 16, scale)
            m = max(abs(x) for x in xs)
            # the exponent is ceil(log2(max)) of the block maximum (block_fp.py:58); 1e-9 does not move the binade
            e = exact_floor_log2(m) + 1
            ys = [S.block_fp_element_f32(x, e, width) for x in xs]
            out["block_fp"].append({"width": width, "exponent_width": 8, "block": 16, "x": [bits(x) for x in xs],
                                    "y": [frac_bits(y, negative_zero=(y == 0 and x < 0)) for x, y in zip(xs, ys)]})
    for (E, F) in ((4, 3), (5, 2), (2, 1), (2, 3), (3, 2)):
        for scale in (1.0, 0.02):
            xs = safe_block(rng, 32, scale)
            m = max(abs(x) for x in xs)
            emax = (1 << E) - 1 - ((1 << (E - 1)) - 1)
            sh = exact_floor_log2(m) - emax
            ys = []
            for x in xs:
                t = Fraction(x) / Fraction(2) ** sh
                tb = bits(float(t))  # exact: a power-of-two scaling of an fp32 value well inside the normal range
                code = S.minifloat_mx_encode(tb, E, F, True, "rn")
                v, sgn = S.minifloat_mx_decode(code, E, F, True)
                ys.append(frac_bits(v * Fraction(2) ** sh, negative_zero=(v == 0 and sgn == 1)))
            out["mxfp"].append({"block_size": 32, "exp_bits": E, "frac_bits": F, "scale_byte": sh + 127,
                                "x": [bits(x) for x in xs], "y": ys})
    # block floating point on bf16 tensors (the headline configuration: width 8, exponent width 8, blocks of 16, and a
    # narrower one).  Values are bf16 bit patterns.  The only rounding to the dtype that changes a value is that of
    # |x| + 1e-9 (S.store: fp32 sum, then bf16); 2^e, the scalings by powers of two and the final product are exact.
    # Block maxima sit in the upper 70 % of their binade, where log2 rounded to bf16 cannot reach the next integer.
    import numpy as np

    def bf16_bits(v):
        b = bits(v)
        assert b & 0xFFFF == 0, v
        return b >> 16

    out["block_fp_bf16"] = []
    for width in (8, 6):
        for scale in (1.0, 50.0, 0.003):
            while True:
                xs = [float(S.round_to(np.float64(rng.gauss(0.0, 1.0) * scale), "bf16")) for _ in range(16)]
                if scale == 50.0:
                    xs[3], xs[7], xs[11] = 0.0, -0.0, float(S.round_to(np.float64(3e-9), "bf16"))
                m = max(abs(x) for x in xs)
                if 1.3 < m / 2.0 ** exact_floor_log2(m) < 1.95:
                    break
            e = exact_floor_log2(m) + 1
            ys = []
            for x in xs:
                if abs(x) <= float(S.round_to(np.float64(1e-8), "bf16")):   # isclose(x, 0): passed through, -0 -> +0
                    ys.append(bf16_bits(abs(x)) if x == 0 else bf16_bits(x))
                    continue
                v = Fraction(float(S.store(np.float64(abs(x)) + S.EPS_F32, "bf16")))
                q = min(max(S.rne(v / Fraction(2) ** e * (1 << (width - 1))), 0), (1 << (width - 1)) - 1)
                y = Fraction(q, 1 << (width - 1)) * Fraction(2) ** e
                ys.append(bf16_bits(float(y)) | (0x8000 if x < 0 else 0))
            out["block_fp_bf16"].append({"width": width, "exponent_width": 8, "block": 16,
                                         "x": [bf16_bits(x) | 0 if not (x == 0 and str(x).startswith("-")) else 0x8000 for x in xs],
                                         "y": ys})
    # the bit-level cast of the MX formats in the regions where the source's arithmetic departs from round-to-nearest
    # (carry out of the fraction in odd / even exponent fields, exponent field 0, below 2^-bias, saturation, the low 8
    # mantissa bits dropped before rounding).  Expected values from the value-domain statement in exact rationals
    # (S.minifloat_mx_value), cross-checked here against the integer restatement of the bit fields.
    out["minifloat_mx"] = []
    rng2 = random.Random(77)
    for (E, F) in ((4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2)):
        bias = (1 << (E - 1)) - 1
        for finite in (True, False):
            top = ((1 << E) - 1 if finite else (1 << E) - 2) - bias
            xs = []
            for e in sorted({-bias - 1, -bias, -bias + 1, -bias + 2, 0, top - 1, top, top + 1}):
                if not -126 <= e <= 127:
                    continue
                for frac in (0.0, 1.0 - 2.0 ** -(F + 1), 1.0 - 2.0 ** -(F + 2), 2.0 ** -(F + 1), 2.0 ** -(F + 1) + 2.0 ** -23,
                             2.0 ** -(F + 1) + 2.0 ** -15, 3 * 2.0 ** -(F + 1), rng2.random(), rng2.random()):
                    xs.append(f32((1.0 + frac) * 2.0 ** e))
            xs += [0.0, -0.0, 1e-40, -1e-40, 3.0e38, -3.0e38]
            xs = [x if i % 3 else -x for i, x in enumerate(xs)]
            for mode in ("rn", "ru", "rd", "rz"):
                ys = []
                for x in xs:
                    v, neg = S.minifloat_mx_value(x, E, F, finite, mode)
                    code = S.minifloat_mx_encode(bits(x), E, F, finite, mode)
                    v2, sgn2 = S.minifloat_mx_decode(code, E, F, finite)
                    if v == "inf":
                        assert v2 in ("inf", "-inf"), (x, E, F, finite, mode)
                        ys.append(0xFF800000 if neg else 0x7F800000)
                        continue
                    assert abs(v2) == v and bool(sgn2) == bool(neg), (x, E, F, finite, mode, v, v2)
                    ys.append(frac_bits(v, negative_zero=(v == 0 and neg)) | (0x80000000 if (neg and v != 0) else 0))
                out["minifloat_mx"].append({"exp_bits": E, "frac_bits": F, "is_finite": finite, "round_mode": mode,
                                            "x": [bits(x) for x in xs], "y": ys})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(path, {k: len(v) for k, v in out.items()}, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
