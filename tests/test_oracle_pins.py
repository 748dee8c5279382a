"""Pins for the CPU oracle (no GPU needed).

The reference holds no golden vectors or value-asserting tests for this path, and running it to make vectors
was refused by the environment.  So each oracle function is checked here against something that does not
share its code: exact rational arithmetic on single values (oracle/scalar.py), brute force over the set of
representable values, invariants of the format, and the host library itself for ``log2``.  A dropped term,
wrong sign, wrong rounding rule or transposed blocking fails at least one of these.
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle as O
from oracle import quantizers as OQ
from oracle import scalar as S
from helpers import adversarial, adversarial_fp32_bits, fp32_from_bits


def exact_log2_parts(v: float):
    """(k, is_power_of_two) with 2^k <= v < 2^(k+1)"""
    m, e = math.frexp(v)
    return e - 1, m == 0.5


def far_from_pow2(v: float, margin: float = 2e-4) -> bool:
    """The library's rounded log2 can only land on the wrong integer for values close to a power of two:
    within ~1e-4 relative in fp32; in bf16, whose log2 result keeps 8 bits, within 25 % above one."""
    m, _ = math.frexp(v)
    return 0.5 * (1 + margin) < m < 1.0 - min(margin, 0.1) or m == 0.5


# ------------------------------------------------------------------ fixed point
@pytest.mark.parametrize("width,frac,signed", [(8, 4, True), (8, 0, True), (4, 6, True), (8, -2, True), (8, 4, False), (12, None, True)])
def test_integer_closed_form(width, frac, signed):
    rng = np.random.default_rng(1)
    x = fp32_from_bits(adversarial_fp32_bits(rng, 3000))
    x = torch.where(torch.isfinite(x) & (x.abs() < 1e30), x, torch.zeros_like(x))
    x = torch.cat([x, torch.randn(2000) * 4, (torch.arange(-600, 600).float() + 0.5) / 2 ** (frac if frac is not None else width // 2)])
    f = frac if frac is not None else width // 2
    for fn, fl in ((O.integer_quantizer, False), (O.integer_floor_quantizer, True)):
        y = fn(x, width, frac, signed)
        for xi, yi in zip(x.tolist(), y.tolist()):
            assert Fraction(yi) == S.integer_quantize(xi, width, f, signed, fl), (xi, yi)


def test_integer_is_idempotent_and_monotone():
    x = torch.randn(10000) * 5
    y = O.integer_quantizer(x, 8, 4)
    assert torch.equal(O.integer_quantizer(y, 8, 4), y)
    xs, _ = torch.sort(x)
    ys = O.integer_quantizer(xs, 8, 4)
    assert bool((ys[1:] >= ys[:-1]).all())


# ------------------------------------------------------------------ MXINT
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,bits,sbits", [(32, 8, 8), (16, 4, 8), (8, 6, 4)])
def test_mxint_closed_form(dtype, B, bits, sbits):
    rng = np.random.default_rng(2)
    x = adversarial(rng, (40, 4 * B), dtype, block=B)
    x = torch.where(x.float().abs() < 1e30, x, torch.zeros_like(x))
    y = O.mxint_quantizer(x, B, bits, scale_bits=sbits)
    xb = x.reshape(-1, B)
    yb = y.reshape(-1, B)
    tiny = torch.finfo(dtype).tiny
    for r in range(xb.shape[0]):
        mx = max(float(xb[r].float().abs().max()), tiny)
        k_lib = int(torch.tensor([mx], dtype=dtype).log2().ceil().item())  # the library's own rounding
        kx, p2 = exact_log2_parts(mx)
        k_exact = kx if p2 else kx + 1
        if far_from_pow2(mx, 2e-4 if dtype == torch.float32 else 0.25):
            assert k_lib == k_exact, (mx, k_lib, k_exact)  # textbook ceil(log2) away from powers of two
        assert k_lib in (k_exact, k_exact - 1)
        want = S.mxint_block(xb[r].float().tolist(), k_lib, bits, sbits)
        got = yb[r].float().tolist()
        for w, g, xi in zip(want, got, xb[r].float().tolist()):
            # exact unless the result is subnormal in the dtype (then it is the correctly rounded value)
            if w != 0 and abs(w) < Fraction(2) ** -120:
                continue
            assert Fraction(g) == w, (xi, mx, k_lib, g, float(w))


def test_mxint_invariants_and_known_answers():
    x = torch.randn(512, 32)
    y = O.mxint_quantizer(x, 32, 8)
    mx = x.abs().amax(1, keepdim=True)
    k = torch.ceil(torch.log2(mx))
    grid = 2.0 ** (k - 7)
    assert torch.equal(torch.round(y / grid) * grid, y)  # every output is on the block's 2^(k-7) grid
    assert bool(((y / grid) >= -128).all()) and bool(((y / grid) <= 127).all())
    assert bool(((y - x).abs() <= grid / 2 + (x.abs() >= mx) * grid).all())  # half-step error, one step at the clamped top
    # values already on the grid come back unchanged, unless the quantized maximum is exactly a power of two
    # (then the second pass picks a smaller exponent and the top code saturates)
    ymax = y.abs().amax(1)
    keep = torch.frexp(ymax)[0] != 0.5
    assert int(keep.sum()) > 400
    assert torch.equal(O.mxint_quantizer(y, 32, 8)[keep], y[keep])
    # a block whose maximum is exactly 2^k: +2^k saturates at 127/128 * 2^k, -2^k is representable
    blk = torch.zeros(2, 32)
    blk[0, 0], blk[0, 1], blk[0, 2] = 4.0, -4.0, 1.0
    blk[1, 0], blk[1, 1] = 0.3, -0.0001
    out = O.mxint_quantizer(blk, 32, 8)
    assert out[0, 0].item() == 127 / 128 * 4 and out[0, 1].item() == -4.0 and out[0, 2].item() == 1.0
    assert out[1, 1].item() == 0.0 and math.copysign(1.0, out[1, 1].item()) == -1.0  # negative underflow keeps -0.0
    # all-zero block: exponent comes from finfo.tiny, result is zero
    assert torch.equal(O.mxint_quantizer(torch.zeros(1, 32), 32, 8), torch.zeros(1, 32))


def test_mxint_block_dim_is_a_transpose():
    x = torch.randn(6, 64, 5)
    a = O.mxint_quantizer(x, 32, 8, block_dim=1)
    b = O.mxint_quantizer(x.transpose(1, 2).contiguous(), 32, 8, block_dim=-1).transpose(1, 2)
    assert torch.equal(a, b)


# ------------------------------------------------------------------ block floating point
def brute_force_tiles(shape, b0, b1):
    """tile id of every element of [batch, rows, cols] by explicit loops"""
    batch, rows, cols = shape
    tr, tc = -(-rows // b0), -(-cols // b1)
    tid = np.empty(shape, dtype=np.int64)
    for b in range(batch):
        for r in range(rows):
            for c in range(cols):
                tid[b, r, c] = (b * tr + r // b0) * tc + c // b1
    return tid


@pytest.mark.parametrize("shape,kw,geom", [
    ((2, 5, 40), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[2, 16], skip_first_dim=True), (2, 5, 40, 2, 16)),
    ((12, 40), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[4, 16], skip_first_dim=False), (1, 12, 40, 4, 16)),
    ((5, 50), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=True), (1, 5, 50, 1, 16)),
    ((33, 48), dict(width=6, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=False), (1, 33, 48, 33, 16)),
    ((37,), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=False), (1, 1, 37, 1, 16)),
    ((2, 4, 48), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=True), (2, 4, 48, 4, 16)),
])
def test_block_fp_closed_form_fp32(shape, kw, geom):
    """fp32: blocking by brute-force index map, element value by exact rational arithmetic."""
    from mase_amd.quantizers._ops import block_fp_geometry

    assert block_fp_geometry(shape, kw["block_size"], kw["skip_first_dim"])[:5] == geom
    rng = np.random.default_rng(3)
    x = torch.from_numpy(rng.standard_normal(int(np.prod(shape))).astype(np.float32)).reshape(shape)
    x.view(-1)[::7] *= 30
    x.view(-1)[3::11] = 0
    x.view(-1)[5::13] = 3e-9
    y = O.block_fp_quantizer(x.clone(), **kw)
    batch, rows, cols, b0, b1 = geom
    tid = brute_force_tiles((batch, rows, cols), b0, b1).reshape(-1)
    xf = x.reshape(-1).tolist()
    yf = y.reshape(-1).tolist()
    tmax = {}
    for t, v in zip(tid, xf):
        tmax[t] = max(tmax.get(t, 0.0), abs(v))
    bias = 127
    for t, xi, yi in zip(tid, xf, yf):
        if abs(xi) <= 1e-8:
            assert yi == xi  # isclose passthrough
            continue
        mx = tmax[t]
        kx, p2 = exact_log2_parts(mx)
        if not far_from_pow2(mx):
            continue
        e = min(max(kx if p2 else kx + 1, -bias), 255 - bias)
        assert Fraction(yi) == S.block_fp_element_f32(xi, e, kw["width"]), (xi, mx, e, yi)


def test_block_fp_zero_tiles_do_not_leak():
    """the substitute exponent for all-zero tiles (block_fp.py:40-44) must not influence any output"""
    x = torch.randn(4, 64)
    x[1] = 0
    a = O.block_fp_quantizer(x.clone(), 8, 8, None, [16], True)
    x2 = x.clone()
    x2[3] *= 1e-20  # changes the smallest non-zero block maximum, i.e. the substitute
    b = O.block_fp_quantizer(x2.clone(), 8, 8, None, [16], True)
    assert torch.equal(a[:3], b[:3]) and torch.equal(a[1], torch.zeros(64))


# ------------------------------------------------------------------ bit-level minifloat
MF = [(4, 3, True), (5, 2, True), (2, 1, True), (2, 3, True), (3, 2, True), (1, 2, True), (4, 3, False), (5, 2, False), (5, 10, False)]


@pytest.mark.parametrize("E,F,finite", MF)
def test_minifloat_mx_matches_scalar_restatement(E, F, finite):
    rng = np.random.default_rng(E * 16 + F)
    bits = np.concatenate([adversarial_fp32_bits(rng, 6000), (np.arange(0, 65536, 5, dtype=np.uint32) << 16)])
    x = fp32_from_bits(bits)
    for rm in ("rn", "ru", "rd", "rz"):
        codes = OQ.minifloat_mx_extract(x, E, F, finite, rm).view(torch.int16).numpy().view(np.uint16)
        dec = OQ.minifloat_mx_compose(torch.from_numpy(codes.view(np.int16)).view(torch.uint16), E, F, finite, torch.float32)
        for b, c, d in zip(bits.tolist(), codes.tolist(), dec.tolist()):
            ab = b & 0x7FFFFFFF
            if finite and ab >= 0x7F800000:
                continue  # Inf/NaN into a format without them: unspecified
            assert c == S.minifloat_mx_encode(b, E, F, finite, rm), (hex(b), rm, c)
            v, sgn = S.minifloat_mx_decode(c, E, F, finite)
            if isinstance(v, str):
                assert (v == "nan" and d != d) or (v == "inf" and d == math.inf) or (v == "-inf" and d == -math.inf)
            else:
                assert Fraction(d) == v and (d != 0 or math.copysign(1, d) == (-1 if sgn else 1))


@pytest.mark.parametrize("E,F", [(4, 3), (5, 2), (2, 1), (2, 3), (3, 2)])
def test_minifloat_mx_is_nearest_value_away_from_the_quirks(E, F):
    """Finite format, round-to-nearest: outside the source-specific regions (carry out of the fraction,
    format subnormals, overflow, underflow) the result must be the representable value nearest to the input
    whose low 8 mantissa bits were dropped, ties to even."""
    reps = S.minifloat_representable(E, F, True)
    bias = (1 << (E - 1)) - 1
    rng = np.random.default_rng(5)
    lo_e, hi_e = 1 - bias, (1 << E) - 1 - bias
    n = 4000
    e = rng.integers(lo_e, hi_e + 1, size=n)
    man = rng.integers(0, 1 << 23, size=n).astype(np.uint32)
    man[::5] &= np.uint32(0x7F8000)  # few significant bits: exact ties after the 8-bit truncation
    bits = (((e + 127).astype(np.uint32)) << 23) | man
    x = fp32_from_bits(bits)
    y = O.minifloat_quantizer_sim(x, E, F, True, "rn").tolist()
    checked = 0
    for b, yi in zip(bits.tolist(), y):
        m15 = (b & 0x7FFFFF) >> 8
        if S.rne(Fraction(m15, 1 << (15 - F))) == (1 << F):
            continue  # carry region (source-specific)
        xt = Fraction(S.bits_f32(b & 0xFFFFFF00))
        best = min(reps, key=lambda r: (abs(r - xt), 0))
        ties = [r for r in reps if abs(r - xt) == abs(best - xt)]
        if len(ties) == 2:  # tie: even fraction field wins
            best = [r for r in ties if (r / (Fraction(2) ** (exact_log2_parts(float(r))[0] - F))).numerator % 2 == 0][0]
        assert Fraction(yi) == best, (hex(b), yi, float(best))
        checked += 1
    assert checked > n // 2


def test_minifloat_mx_documented_quirks():
    """The source-specific behaviours on hand-picked points (their value-domain closed form is swept exhaustively in
    test_minifloat_mx_value_pins.py)."""
    q = lambda v, E, F: O.minifloat_quantizer_sim(torch.tensor([v], dtype=torch.float32), E, F, True, "rn").item()
    assert q(500.0, 4, 3) == 256.0     # [496,512): fraction rounds to 2^F, exponent field 15 is odd -> carry lost
    assert q(480.0, 4, 3) == 480.0     # all-finite e4m3 tops out at 480, not 448
    assert q(1e9, 4, 3) == 480.0
    assert q(7.5, 2, 1) == 4.0         # e2m1 [7,8): same lost carry
    assert q(2.0 ** -7 * 1.03, 4, 3) == 0.0   # exponent field 0 with fraction 0 decodes to zero
    assert math.copysign(1, q(-1e-30, 4, 3)) == -1.0  # sign survives underflow


# ------------------------------------------------------------------ MXFP
@pytest.mark.parametrize("E,F", [(4, 3), (2, 1), (5, 2), (3, 2)])
def test_mxfp_closed_form(E, F):
    rng = np.random.default_rng(9)
    x = adversarial(rng, (24, 64), torch.float32, block=32)
    x = torch.where(x.abs() < 1e30, x, torch.zeros_like(x))
    y = O.mxfp_quantizer(x, 32, E, F)
    sc, el = OQ.mxfp_components(x.flatten(), 32, E, F)
    emax = (1 << E) - 1 - ((1 << (E - 1)) - 1)
    xb, yb = x.reshape(-1, 32), y.reshape(-1, 32)
    for r in range(xb.shape[0]):
        vals = [0.0 if (S.f32_bits(v) & 0x7F800000) == 0 else v for v in xb[r].tolist()]
        mx = max(abs(v) for v in vals)
        if mx == 0:
            assert int(sc[r]) == 0 and torch.equal(yb[r], torch.zeros(32))
            continue
        k_lib = int(torch.tensor([mx]).log2().floor().item())
        kx, _ = exact_log2_parts(mx)
        if far_from_pow2(mx):
            assert k_lib == kx
        sh = min(max(k_lib - emax, -127), 128)
        assert int(sc[r]) == sh + 127
        for v, yi, c in zip(vals, yb[r].tolist(), el[r].tolist()):
            scaled = float(np.float32(v) / np.float32(2.0) ** np.float32(sh)) if -126 <= sh <= 127 else None
            if scaled is None:
                continue
            code = S.minifloat_mx_encode(S.f32_bits(scaled), E, F, True, "rn")
            assert c == code
            d, _ = S.minifloat_mx_decode(code, E, F, True)
            assert Fraction(yi) == d * Fraction(2) ** sh


# ------------------------------------------------------------------ element-wise minifloat (fp32 closed form)
@pytest.mark.parametrize("w,ew", [(8, 4), (8, 5), (6, 3)])
def test_minifloat_denorm_ieee_closed_form_fp32(w, ew):
    rng = np.random.default_rng(12)
    x = torch.from_numpy((rng.standard_normal(3000) * np.exp(rng.uniform(-8, 8, 3000))).astype(np.float32))
    mb = w - ew - 1
    bias = 2 ** (ew - 1) - 1
    yd = O.minifloat_denorm_quantizer(x, w, ew).tolist()
    yi = O.minifloat_ieee_quantizer(x, w, ew).tolist()
    n = 0
    for xi, d, i in zip(x.tolist(), yd, yi):
        a = abs(xi)
        v = S.bits_f32(S.f32_bits(a + S.bits_f32(S.f32_bits(1e-9))))
        if a <= 1e-8 or not far_from_pow2(v):
            continue
        kx, p2 = exact_log2_parts(v)
        # denorm: exponent = ceil(log2), mantissa in [0,1) with mb bits, no implicit one
        e = min(max(kx if p2 else kx + 1, -bias), 2 ** ew - 1 - bias)
        q = min(max(S.rne(Fraction(a) / Fraction(2) ** e * 2 ** mb), 0), 2 ** mb - 1)
        want = Fraction(q, 2 ** mb) * Fraction(2) ** e
        assert Fraction(abs(d)) == want and (d == 0 or (d < 0) == (xi < 0))
        # ieee: exponent = floor(log2); implicit one unless the exponent clamps to -bias
        e = min(max(kx, -bias), 2 ** ew - 1 - bias)
        man = Fraction(a) / Fraction(2) ** e
        if e != -bias:
            q = min(max(S.rne(man * 2 ** mb - 2 ** mb), 0), 2 ** mb - 1)
            want = (1 + Fraction(q, 2 ** mb)) * Fraction(2) ** e
        else:
            q = min(max(S.rne(man * 2 ** mb / 2), 0), 2 ** mb - 1)
            want = Fraction(q, 2 ** mb) * 2 * Fraction(2) ** e
        assert Fraction(abs(i)) == want
        n += 1
    assert n > 2000


# ------------------------------------------------------------------ 16-bit tensors: explicit-rounding models
_T16 = {"bf16": torch.bfloat16, "f16": torch.float16}


def all_16bit_values(fmt, finite_only=True):
    bits16 = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    t = bits16.view(_T16[fmt])
    if finite_only:
        t = t[torch.isfinite(t.float())]
    return t


def lib_log2(fmt):
    return lambda v: torch.from_numpy(np.asarray(v)).to(_T16[fmt]).log2().double().numpy()


def lib_close(t):
    return torch.isclose(t, torch.tensor([0.0], dtype=t.dtype)).numpy()


def same_values(got: torch.Tensor, want: np.ndarray):
    """bit-level equality of a 16-bit tensor with float64 model values (signed zeros told apart, NaN == NaN)"""
    g = got.double().numpy()
    ok = ((g == want) & (np.signbit(g) == np.signbit(want))) | (np.isnan(g) & np.isnan(want))
    return ok


def test_explicit_rounding_helper_is_round_to_nearest_even():
    """the model's own rounding routine against exact rational arithmetic (ties, subnormals, overflow)"""
    rng = np.random.default_rng(5)
    for fmt, (p, qmin, vmax) in S.FMT.items():
        vals = list((rng.standard_normal(300) * np.exp(rng.uniform(-60, 40, 300))).astype(np.float64))
        vals += [np.ldexp(1.0 + (2 * k + 1) * 2.0 ** -p, e) for k in range(4) for e in (-3, 0, 7)]       # exact ties
        vals += [np.ldexp(float(k) + 0.5, qmin) for k in range(6)] + [np.ldexp(0.5, qmin), np.ldexp(0.25, qmin)]
        vals += [vmax, np.nextafter(vmax, np.inf), vmax + np.ldexp(1.0, int(np.log2(vmax)) - p), vmax * 1.1]
        got = S.round_to(np.array(vals), fmt)
        for v, g in zip(vals, got):
            fr = Fraction(float(v))
            k = 0 if fr == 0 else (abs(fr).numerator.bit_length() - abs(fr).denominator.bit_length())
            while Fraction(2) ** k > abs(fr):
                k -= 1
            while Fraction(2) ** (k + 1) <= abs(fr):
                k += 1
            qe = max(k + 1 - p, qmin)
            want = Fraction(S.rne(fr / Fraction(2) ** qe)) * Fraction(2) ** qe
            if abs(want) > Fraction(vmax):
                assert np.isinf(g) and (g > 0) == (fr > 0), (fmt, v, g)
            else:
                assert Fraction(float(g)) == want, (fmt, v, g, float(want))


@pytest.mark.parametrize("fmt", ["bf16", "f16"])
@pytest.mark.parametrize("width", [8, 6, 9])
def test_block_fp_16bit_every_value_as_block_maximum_and_as_element(fmt, width):
    """block_fp_quantizer on bf16 / fp16 (width 8 on bf16 is the headline configuration): the oracle against (1) the
    op-by-op model with every rounding to the dtype written out and (2), where it applies, the closed form with the
    single rounding of |x| + 1e-9; exponents from the library's own log2 in the dtype.  Every finite 16-bit value
    serves once as the maximum of a block and once as an element of blocks with a larger maximum."""
    T = _T16[fmt]
    vals = all_16bit_values(fmt)
    n = vals.numel()
    # (a) every value as block maximum: element 0 is the value, the others are fixed fractions of it
    fr = torch.tensor([1.0, 0.5, -0.75, 0.3, -0.011, 0.99, 1e-3, -1.0, 0.0, 0.66, -0.2, 0.127, 0.9, -0.45, 2.0 ** -9, 0.07])
    blocks_a = (vals.float()[:, None] * fr[None, :]).to(T)
    # (b) every value as an element: 15 values per block, the block maximum a fixed larger value
    cases = [blocks_a]
    for mx in ((1.0, 200.0, 3e-4, 40000.0) if fmt == "f16" else (1.0, 200.0, 3e-4, 7e20, 1e-30)):
        sel = vals[vals.float().abs() <= mx]
        sel = sel[: sel.numel() // 15 * 15].reshape(-1, 15)
        cases.append(torch.cat((torch.full((sel.shape[0], 1), mx).to(T), sel), dim=1))
    checked = closed = 0
    for blocks in cases:
        got = O.block_fp_quantizer(blocks.clone(), width, 8, None, [16], True)
        bmax = blocks.float().abs().amax(1, keepdim=True).to(T)
        with np.errstate(divide="ignore"):
            lg = np.ceil(lib_log2(fmt)(bmax.double().numpy()))               # -inf for an all-zero block
        lg = np.broadcast_to(lg, blocks.shape).copy()
        close = lib_close(blocks)
        x = blocks.double().numpy()
        lg[np.isneginf(lg)] = 0.0   # all-zero blocks: every element takes the isclose branch, the exponent is moot
        want = S.block_fp_model(x, lg, close, width, 8, fmt)
        ok = same_values(got, want)
        assert ok.all(), (fmt, width, int((~ok).sum()), x[~ok][:4], got.double().numpy()[~ok][:4], want[~ok][:4])
        checked += ok.size
        # closed form: exponent inside the range where 2^e and the scalings are exact in the dtype
        e = np.clip(lg, -127, 128)
        lo, hi = ((-14 + width, 15) if fmt == "f16" else (-120, 120))
        dom = (~close) & (e >= lo) & (e <= hi) & (np.abs(x) < np.ldexp(1.0, e.astype(np.int64) + 1))
        cf = S.block_fp_closed_form(x[dom], e[dom], width, fmt)
        g = got.double().numpy()[dom]
        assert ((g == cf) | ((g == 0) & (cf == 0))).all(), (fmt, width)
        closed += int(dom.sum())
    assert checked > n * 17 and closed > n * 8, (checked, closed, n)


@pytest.mark.parametrize("fmt", ["bf16", "f16"])
@pytest.mark.parametrize("w,ew", [(8, 4), (8, 5), (6, 3)])
def test_minifloat_denorm_ieee_16bit_exhaustive(fmt, w, ew):
    """minifloat_denorm / ieee on bf16 and fp16 tensors, every finite 16-bit input: the oracle against the op-by-op
    model in which each op's result is rounded to fp32 and then to the dtype explicitly (log2 and isclose are the
    library's own, evaluated in the dtype)"""
    vals = all_16bit_values(fmt)
    x = vals.double().numpy()
    close = lib_close(vals.abs())
    for ieee, fn in ((False, O.minifloat_denorm_quantizer), (True, O.minifloat_ieee_quantizer)):
        got = fn(vals.clone(), w, ew)
        want = S.minifloat_model(x, lib_log2(fmt), close, w, ew, fmt, ieee)
        ok = same_values(got, want)
        assert ok.all(), (fmt, w, ew, ieee, int((~ok).sum()), x[~ok][:5], got.double().numpy()[~ok][:5], want[~ok][:5])
        # the model reduces to the textbook value away from the library's log2 thresholds: spot-check in exact arithmetic
        mb, bias = w - ew - 1, 2 ** (ew - 1) - 1
        idx = np.flatnonzero(~close & (np.abs(x) > 2.0 ** (-bias + 1)) & (np.abs(x) < 2.0 ** (2 ** ew - 2 - bias)))[::97]
        for i in idx:
            a = abs(float(x[i]))
            if not far_from_pow2(a, 0.02):
                continue
            kx, p2 = exact_log2_parts(a)
            if ieee:
                q = min(max(S.rne(Fraction(a) / Fraction(2) ** kx * 2 ** mb - 2 ** mb), 0), 2 ** mb - 1)
                expect = (1 + Fraction(q, 2 ** mb)) * Fraction(2) ** kx
            else:
                e = kx if p2 else kx + 1
                q = min(max(S.rne(Fraction(a) / Fraction(2) ** e * 2 ** mb), 0), 2 ** mb - 1)
                expect = Fraction(q, 2 ** mb) * Fraction(2) ** e
            assert Fraction(abs(float(want[i]))) == expect, (fmt, w, ew, ieee, a)


@pytest.mark.parametrize("E,F", [(4, 3), (5, 2), (2, 1), (2, 3), (3, 2), (1, 2), (5, 8), (6, 9), (5, 10)])
def test_minifloat_mx_invariants_fixed_by_the_format(E, F):
    """what the format itself fixes, whatever the source-specific roundings do: every code fits in 1 + E + F bits, for
    any input and rounding mode; every code with a non-zero exponent field decodes to a value that encodes back to
    the same code (decode after encode is the identity on the format's normal values).  Codes with exponent field 0
    are the source-specific part (values below 2^-bias are flushed, the negative-zero code becomes the zero code):
    for those the vectorised restatement is held to the scalar one."""
    from helpers import adversarial_fp32_bits, fp32_from_bits

    rng = np.random.default_rng(E * 16 + F)
    x = fp32_from_bits(adversarial_fp32_bits(rng, 40000, finite_only=False))
    for finite in (True, False):
        for mode in ("rn", "ru", "rd", "rz"):
            codes = O.minifloat_mx_extract(x, E, F, finite, mode)
            assert int(codes.to(torch.int32).max()) < (1 << (1 + E + F)) and int(codes.to(torch.int32).min()) >= 0
    all_codes = torch.arange(0, 1 << (1 + E + F), dtype=torch.int32).to(torch.uint16)
    for finite in (True, False):
        dec = O.minifloat_mx_compose(all_codes.clone(), E, F, finite, torch.float32)
        back = O.minifloat_mx_extract(dec, E, F, finite, "rn").to(torch.int32)
        want = all_codes.to(torch.int32)
        xe = (want >> F) & ((1 << E) - 1)
        top = (1 << E) - 1
        expect = want.clone()
        for i in range(want.numel()):
            v, sgn = S.minifloat_mx_decode(int(want[i]), E, F, finite)
            if isinstance(v, str):
                continue
            expect[i] = S.minifloat_mx_encode(S.f32_bits(float(v)) | ((sgn << 31) if v == 0 else 0), E, F, finite, "rn")
        finite_code = torch.tensor([not isinstance(S.minifloat_mx_decode(int(c), E, F, finite)[0], str) for c in want])
        assert torch.equal(back[finite_code], expect[finite_code])
        stable = finite_code & (xe > 0) & ((xe < top) | finite)
        assert torch.equal(back[stable], want[stable]), "normal codes must survive decode -> encode"


# ------------------------------------------------------------------ Linear glue
def test_linear_forwards_are_f_linear_of_quantized_operands():
    torch.manual_seed(0)
    x, w, b = torch.randn(4, 64), torch.randn(8, 64) * 0.02, torch.randn(8)
    cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}
    from oracle import linear as OL

    qw, qb = OL.mxint_prepare_weights(w, b, cfg)
    assert torch.equal(qw, O.mxint_quantizer(w, 32, 8, block_dim=1)) and qb is b
    y = OL.linear_mxint_forward(x, qw, qb, cfg)
    assert torch.equal(y, torch.nn.functional.linear(O.mxint_quantizer(x, 32, 8), qw, b))
    assert torch.equal(OL.linear_mxint_forward(x, qw, qb, {**cfg, "bypass": True}), torch.nn.functional.linear(x, qw, b))


# ------------------------------------------------------------------------------------------------
# clip search (quantile_search=True without calibration activations)
# ------------------------------------------------------------------------------------------------
def _exact_quantile(sorted_vals, q: float):
    """the library's linear interpolation as the kernels restate it: fp32 rank and weight, one fused multiply-add"""
    n = len(sorted_vals)
    rank = np.float32(q) * np.float32(n - 1)
    lo = int(math.floor(rank))
    hi = int(math.ceil(rank))
    w = np.float32(rank - np.float32(lo))
    a, b = Fraction(float(sorted_vals[lo])), Fraction(float(sorted_vals[hi]))
    diff = Fraction(float(np.float32(float(b - a))))  # b - a rounded to fp32
    if w < 0.5:
        exact = Fraction(float(w)) * diff + a
    else:
        exact = Fraction(float(np.float32(w - np.float32(1)))) * diff + b
    # one rounding of the exact result to fp32 (float() of a Fraction rounds correctly to double first, which is
    # harmless here only if the double is not a tie of fp32: compare in rationals instead)
    lo32 = np.float32(float(exact))
    cands = [lo32, np.nextafter(lo32, np.float32(np.inf)), np.nextafter(lo32, np.float32(-np.inf))]
    return min(cands, key=lambda c: (abs(Fraction(float(c)) - exact), int(np.float32(c).view(np.uint32)) & 1))


def test_library_quantile_is_the_fused_interpolation():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(40, 32, generator=g).abs() * torch.exp2(torch.randint(-20, 20, (40, 1), generator=g).float())
    got = x.quantile(torch.tensor(O.CLIP_PERCENTILES, dtype=torch.float32), dim=1)  # [11, 40]
    s = x.sort(dim=1).values.numpy()
    for i, q in enumerate(O.CLIP_PERCENTILES):
        for r in range(x.shape[0]):
            assert np.float32(got[i, r].item()) == _exact_quantile(s[r], q), (q, r)
    assert torch.equal(x.quantile(0.93, dim=1), got[5])  # the scalar overload used by the MXFP extraction


@pytest.mark.parametrize("bits", [8, 4])
def test_mxint_clip_search_picks_the_candidate_with_the_smallest_exact_error(bits):
    g = torch.Generator().manual_seed(bits)
    x = torch.randn(24, 32, generator=g) * 0.1
    x[::3, 0] = 0.2505  # a maximum just above a power of two: clipping it costs little, the finer scale gains more
    out, pick, err, cand = O.mxint_clip_search(x, 32, bits)
    assert cand.shape == (11, 24, 32) and err.shape == (11, 24)
    assert torch.equal(cand[0].reshape(x.shape), O.mxint_quantizer(x, 32, bits))  # percentile 1.0 is the plain quantizer
    assert torch.equal(out, cand[pick, torch.arange(24)].reshape(x.shape))
    assert int((pick != 0).sum()) >= (4 if bits == 4 else 1)
    s = x.abs().sort(dim=1).values.numpy()
    for r in range(24):
        xs = [float(v) for v in x[r]]
        exact = []
        for i, q in enumerate(O.CLIP_PERCENTILES):
            mx = max(float(_exact_quantile(s[r], q)), float(torch.finfo(torch.float32).tiny))
            k, is_pow2 = exact_log2_parts(mx)
            if not is_pow2:
                if not far_from_pow2(mx):
                    break
                k += 1
            ys = S.mxint_block(xs, k, bits)
            assert [float(y) for y in ys] == cand[i, r].tolist(), (r, i)
            exact.append(sum((y - Fraction(v)) ** 2 for y, v in zip(ys, xs)))
        else:
            best = min(exact)
            first = exact.index(best)
            chosen = exact[int(pick[r])]
            assert chosen <= best * (1 + Fraction(1, 1 << 20)), (r, int(pick[r]), first)
            if all(e == best or e > best * (1 + Fraction(1, 1 << 18)) for e in exact):
                assert int(pick[r]) == first  # no near-tie: the first minimum, as argmin returns it


def test_mxfp_clip_search_score_is_on_the_integer_codes():
    """mxfp/mxfp.py:58-62: the score compares x with code / 2^(F-1) * (2^(scale-127) in uint8 arithmetic)"""
    g = torch.Generator().manual_seed(4)
    E, F = 2, 1
    x = torch.randn(16, 32, generator=g) * 30
    x[:, 0] = 100.0  # scale byte 127 + 6 - 2 = 131 for percentile 1.0
    x[5:8] *= 2.0 ** -10  # scale bytes below 127: every candidate scores sum(x^2)
    out, pick, err, cand = O.mxfp_clip_search(x, 32, E, F)
    assert torch.equal(cand[0].reshape(x.shape), O.mxfp_quantizer(x, 32, E, F))
    assert torch.equal(out, cand[pick, torch.arange(16)].reshape(x.shape))
    assert bool((pick[5:8] == 0).all()) and int((pick != 0).sum()) >= 4
    flat = x.reshape(-1)
    for i, q in enumerate(O.CLIP_PERCENTILES):
        sc, el = O.mxfp_components(flat, 32, E, F, percentile=q)
        for r in range(16):
            s = int(sc[r, 0])
            pw = (1 << (s - 127)) if 127 <= s <= 134 else 0
            score = sum((Fraction(int(c)) * pw - Fraction(float(v))) ** 2 for c, v in zip(el[r].tolist(), x[r].tolist()))
            assert abs(float(err[i, r]) - float(score)) <= float(score) * 1e-5 + 1e-30, (i, r)
    # the winner is the first strictly smaller score
    for r in range(16):
        best, who = float("inf"), 0
        for i in range(11):
            if float(err[i, r]) < best:
                best, who = float(err[i, r]), i
        assert int(pick[r]) == who


# ------------------------------------------------------------------------------------------------
# GPTQ
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", ["mxint", "mxfp"])
def test_clip_search_scored_on_calibration_outputs_is_the_gram_matrix_form(fmt):
    """quantile_search with act_tensor: the error of candidate p for weight row h is the sum over calibration batches of
    sqrt(d^T G d), d = candidate - row (for MXFP: the scored values - row), G = the batch's Gram matrix of activations.
    Evaluated in float64 from that formula, independently of the oracle's matmul / einsum / norm calls; the oracle's
    pick must be the formula's minimum (first minimum for MXINT, strict replacement in percentile order for MXFP),
    except where the two best errors agree to within float32 rounding."""
    g = torch.Generator().manual_seed(31)
    B, rows = 32, 64
    w = torch.randn(rows, B, generator=g) * (0.05 if fmt == "mxint" else 30.0)
    w[3, 0] *= 40
    act = torch.randn(5, 24, B, generator=g)
    act[..., 0] *= 0.05
    bsz = 2
    if fmt == "mxint":
        out, pick, err, cand = O.mxint_clip_search(w, B, 4, 1, act_tensor=act, cali_batch_size=bsz)
        scored = cand.double()
    else:
        out, pick, err, cand = O.mxfp_clip_search(w, B, 2, 1, 1, act_tensor=act, cali_batch_size=bsz)
        # the scored values: integer codes times the uint8 power (recomputed here from the components)
        flat = w.reshape(-1)
        scored = []
        for pct in O.CLIP_PERCENTILES:
            sc, el = O.mxfp_components(flat, B, 2, 1, 8, True, "rn", pct)
            e = sc.to(torch.int64) - 127
            unit = torch.where((e >= 0) & (e <= 7), torch.exp2(e.double()), torch.zeros_like(e, dtype=torch.float64))
            scored.append(el.double() / 2 ** (1 - 1) * unit)
        scored = torch.stack(scored)
    exact = torch.zeros(11, rows, dtype=torch.float64)
    for b in range(0, act.shape[0], bsz):
        a = act[b:b + bsz].double().reshape(-1, B)
        G = a.T @ a
        d = scored - w.double()[None]
        exact += torch.sqrt(torch.einsum("phb,bc,phc->ph", d, G, d).clamp_min(0))
    if fmt == "mxint":
        want = exact.argmin(0)
    else:
        want = torch.zeros(rows, dtype=torch.int64)
        best = torch.full((rows,), float("inf"), dtype=torch.float64)
        for p in range(11):
            better = exact[p] < best
            best = torch.where(better, exact[p], best)
            want = torch.where(better, torch.full_like(want, p), want)
    differ = (want != pick).nonzero().flatten()
    for h in differ.tolist():
        a, b = float(exact[want[h], h]), float(exact[pick[h], h])
        assert abs(a - b) <= 1e-5 * max(abs(a), 1e-30), (fmt, h, int(want[h]), int(pick[h]), a, b)
    assert differ.numel() <= rows // 8
    assert int((pick != 0).sum()) > 3
    chosen = cand[pick, torch.arange(rows)]
    assert torch.equal(out, chosen.reshape(out.shape).to(out.dtype))


def _correlated_inputs(g, n, tokens, cols):
    mix = torch.randn(cols, cols, generator=g) * 0.3 + torch.eye(cols)
    return [torch.randn(2, tokens, cols, generator=g) @ mix for _ in range(n)]


def test_gptq_hessian_and_inverse_factor():
    from oracle import gptq as G

    g = torch.Generator().manual_seed(0)
    xs = _correlated_inputs(g, 3, 40, 64)
    H = G.hessian(xs)
    flat = torch.cat([x.reshape(-1, 64) for x in xs]).double()
    want = 2.0 / 6 * flat.t() @ flat  # n counts batch items (6), not tokens: gptq.py:31-36
    assert float((H.double() - want).abs().max() / want.abs().max()) < 1e-5
    U, dead = G.inverse_factor(H)
    assert not bool(dead.any()) and bool((U.tril(-1) == 0).all())
    damped = H.double() + 0.01 * H.diag().double().mean() * torch.eye(64, dtype=torch.float64)
    assert float(((U.double().t() @ U.double()) @ damped - torch.eye(64, dtype=torch.float64)).abs().max()) < 1e-3


@pytest.mark.parametrize("fmt,cfg", [("mxint", {"weight_block_size": 32, "weight_width": 4}),
                                     ("mxfp", {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1})])
def test_gptq_feedback_lowers_the_proxy_loss(fmt, cfg):
    from oracle import gptq as G

    g = torch.Generator().manual_seed(1)
    W = torch.randn(48, 128, generator=g) * 0.05
    # uncorrelated inputs: nothing to feed back, the result is the plain clip-search quantization group by group
    Hd = torch.diag(torch.rand(128, generator=g) + 0.5)
    Q = G.fasterquant(W, Hd, fmt, cfg)
    assert torch.equal(Q, G.quantize_group(W, fmt, cfg, True))
    # correlated inputs: the error feedback must pay off on the calibration data
    H = G.hessian(_correlated_inputs(g, 4, 64, 128))
    Q = G.fasterquant(W, H, fmt, cfg)
    rtn = G.quantize_group(W, fmt, cfg, True)
    assert not torch.equal(Q, rtn)
    assert G.proxy_loss(W, Q, H) < 0.9 * G.proxy_loss(W, rtn, H)
    # a dead column (never active in calibration) is zeroed before quantization (gptq.py:67-69)
    H2 = H.clone()
    H2[5, :] = 0
    H2[:, 5] = 0
    assert bool((G.fasterquant(W, H2, fmt, cfg)[:, 5] == 0).all())


@pytest.mark.parametrize("fmt,cfg", [("mxint", {"weight_block_size": 1, "weight_width": 4}),
                                     ("mxint", {"weight_block_size": 1, "weight_width": 8})])
def test_gptq_with_groups_of_one_column_is_the_textbook_column_update(fmt, cfg):
    """With one column per group nothing of the group-wise simplification is left (inside a group the reference
    divides by the diagonal of the factor's block instead of solving with the block, gptq.py:111-117), and the walk must
    be optimal-brain-surgeon rounding column by column: with H_c the damped Hessian restricted to the columns not yet
    rounded, the error of column c divided by (H_c^-1)[0, 0] is fed into the others through (H_c^-1)[0, 1:].  That is
    evaluated here in float64 with an explicit inverse per column, no Cholesky factor involved."""
    from oracle import gptq as G

    g = torch.Generator().manual_seed(8)
    cols = 7
    W = torch.randn(6, cols, generator=g)
    X = torch.randn(50, cols, generator=g) @ (torch.randn(cols, cols, generator=g) * 0.5 + torch.eye(cols))
    H = G.hessian([X])
    got = G.fasterquant(W, H, fmt, cfg, quant_search=False)
    Hd = H.double() + 0.01 * torch.diagonal(H).double().mean() * torch.eye(cols, dtype=torch.float64)
    Wd = W.double().clone()
    want = torch.zeros_like(Wd)
    for c in range(cols):
        inv = torch.linalg.inv(Hd[c:, c:])
        q = O.mxint_quantizer(Wd[:, c:c + 1].float(), 1, cfg["weight_width"], 1).double()
        want[:, c:c + 1] = q
        Wd[:, c + 1:] -= (Wd[:, c:c + 1] - q) / inv[0, 0] @ inv[0:1, 1:]
    assert float((got.double() - want).abs().max()) == 0.0
    # and a wrong sign of the feed-forward, or the factor transposed, does not give this result
    assert not torch.equal(got, O.mxint_quantizer(W, 1, cfg["weight_width"], 1))
