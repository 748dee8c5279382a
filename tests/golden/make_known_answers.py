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
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(path, {k: len(v) for k, v in out.items()}, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
