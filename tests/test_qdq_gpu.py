"""GPU parity: every quantize-dequantize kernel, called through the package (ctypes -> C ABI -> HIP), must be
bit-exact against the CPU oracle on the same inputs.  -0.0 vs +0.0 counts as a mismatch; NaN matches NaN."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import adversarial, adversarial_fp32_bits, assert_bits_equal, fp32_from_bits

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
_ID = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


@pytest.fixture(scope="module")
def Q(dev):
    import mase_amd.quantizers as q

    return q


def all_16bit(dtype):
    b = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    v = b.view(dtype)
    return torch.where(torch.isfinite(v.float()), v, torch.zeros_like(v))


# ------------------------------------------------------------------ MXINT
@pytest.mark.parametrize("dtype", DTYPES, ids=_ID.get)
@pytest.mark.parametrize("block,bits,sbits", [(32, 8, 8), (16, 8, 8), (32, 4, 8), (8, 6, 8), (4, 8, 8), (2, 8, 8),
                                              (64, 8, 8), (128, 5, 8), (256, 8, 8), (24, 8, 8), (32, 8, 4), (32, 12, 8),
                                              (1024, 8, 8)])
def test_mxint_adversarial(Q, dev, dtype, block, bits, sbits):
    rng = np.random.default_rng(1000 + block * 7 + bits)
    x = adversarial(rng, (96, 3072 // 1), dtype, block=block if 3072 % block == 0 else 32)
    if x.numel() % block:
        x = x.view(-1)[: (x.numel() // block) * block]
    want = O.mxint_quantizer(x, block, bits, scale_bits=sbits)
    got = Q.mxint_quantizer(x.to(dev), block, bits, scale_bits=sbits)
    assert_bits_equal(got, want, f"mxint {dtype} B={block} b={bits} s={sbits}")


@pytest.mark.parametrize("dtype", DTYPES, ids=_ID.get)
def test_mxint_block_dims_and_ragged_rows(Q, dev, dtype):
    rng = np.random.default_rng(7)
    x = adversarial(rng, (6, 64, 40), dtype, block=8)
    for dim, B in [(-1, 8), (1, 32), (0, 2), (2, 20), (-2, 16)]:
        want = O.mxint_quantizer(x, B, 8, block_dim=dim)
        got = Q.mxint_quantizer(x.to(dev), B, 8, block_dim=dim)
        assert_bits_equal(got, want, f"mxint dim={dim} B={B}")
    # last dim not divisible by the block: blocks straddle rows of the flattened tensor
    y = adversarial(rng, (16, 24), dtype, block=8)
    assert_bits_equal(Q.mxint_quantizer(y.to(dev), 32, 8), O.mxint_quantizer(y, 32, 8), "straddling blocks")
    # unaligned view
    z = adversarial(rng, (4, 130), dtype, block=2)[:, 1:129]
    assert_bits_equal(Q.mxint_quantizer(z.to(dev), 32, 8), O.mxint_quantizer(z, 32, 8), "view")
    with pytest.raises(AssertionError):
        Q.mxint_quantizer(torch.zeros(3, 10, device=dev, dtype=dtype), 32, 8)
    assert Q.mxint_quantizer(torch.zeros(0, 32, device=dev, dtype=dtype), 32, 8).shape == (0, 32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=_ID.get)
def test_mxint_every_16bit_value_as_block_max(Q, dev, dtype):
    """Each positive finite value of the dtype is the maximum of one block: exercises every log2 correction."""
    v = all_16bit(dtype)[: 0x7F80 if dtype == torch.bfloat16 else 0x7C00]
    x = (v.float().unsqueeze(1) * torch.linspace(-1, 1, 32).unsqueeze(0)).to(dtype)
    x[:, 31] = v
    want = O.mxint_quantizer(x, 32, 8)
    got = Q.mxint_quantizer(x.to(dev), 32, 8)
    assert_bits_equal(got, want, f"mxint all maxima {dtype}")


def test_mxint_fp32_power_of_two_neighbourhood(Q, dev):
    """Block maxima 2^k (1 +- m ulp), all k, m <= 48: the fp32 log2 corrections."""
    k = torch.arange(-126, 128, dtype=torch.float64)
    rows = []
    for m in list(range(0, 49)):
        rows.append(torch.ldexp(torch.tensor(1.0 + m * 2.0 ** -23, dtype=torch.float64), k.to(torch.int32)))
        rows.append(torch.ldexp(torch.tensor(2.0 - m * 2.0 ** -23, dtype=torch.float64), k.to(torch.int32) - 1))
    mx = torch.cat(rows).to(torch.float32)
    mx = mx[torch.isfinite(mx)]
    x = (mx.unsqueeze(1) * torch.linspace(-0.999, 0.999, 32).unsqueeze(0).float())
    x[:, 5] = -mx
    want = O.mxint_quantizer(x, 32, 8)
    got = Q.mxint_quantizer(x.to(dev), 32, 8)
    assert_bits_equal(got, want, "mxint fp32 pow2 neighbourhood")


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=_ID.get)
@pytest.mark.parametrize("block,bits", [(32, 8), (8, 8), (16, 4), (64, 8), (128, 12), (512, 8), (1024, 8), (4, 8)])
def test_mxint_fp32_in_16bit_out(dev, out_dtype, block, bits):
    """The activation quantizer of an MX Linear on fp32 inputs writes its result in a 16-bit dtype directly
    (``mxint_qdq(..., out_dtype=)``): the oracle's fp32 result converted to that dtype, bit for bit, for blocks that take
    the wide kernel (8 elements per lane) and blocks that do not, a ragged tail, the log2 corrections next to powers of
    two, non-finite blocks and values that overflow fp16"""
    from mase_amd.quantizers import _ops

    rng = np.random.default_rng(77 + block + bits)
    x = adversarial(rng, (96, 3072), torch.float32, block=block if 3072 % block == 0 else 32).reshape(-1)
    k = torch.arange(-100, 100, dtype=torch.int32)
    edge = torch.cat([torch.ldexp(torch.tensor(1.0 + m * 2.0 ** -23, dtype=torch.float64), k) for m in (0, 1, 2, 5, 9)]).float()
    x[: edge.numel()] = edge
    x[5000] = float("inf")
    x[9000] = float("nan")
    x[12000] = 7.0e4   # finite in fp32 and bf16, infinite in fp16
    n = (x.numel() // block) * block - block * 3  # not a multiple of the work-group's 512 elements
    x = x[:n].contiguous()
    want = O.mxint_quantizer(x, block, bits).to(out_dtype)
    got = _ops.mxint_qdq(x.to(dev), block, bits, -1, 8, out_dtype=out_dtype)
    assert_bits_equal(got, want, f"mxint fp32 -> {out_dtype} B={block} b={bits}")


def test_mxint_nonfinite_blocks(Q, dev):
    x = torch.randn(8, 32)
    x[1, 3] = float("inf")
    x[2, 4] = float("nan")
    x[3, 5] = -float("inf")
    x[4, 6] = 3.0e38
    want = O.mxint_quantizer(x, 32, 8)
    got = Q.mxint_quantizer(x.to(dev), 32, 8)
    assert_bits_equal(got, want, "mxint nonfinite")


def test_mxint_packed_components(Q, dev):
    """codes * 2^(scale-134) reproduces the dequantized tensor exactly; codes/scales equal the oracle's."""
    from mase_amd.quantizers import _ops

    rng = np.random.default_rng(11)
    for dtype in DTYPES:
        x = adversarial(rng, (64, 256), dtype, block=32).clamp(-1e4, 1e4)
        deq, codes, scales = _ops.mxint_qdq(x.to(dev), 32, 8, -1, 8, pack=True)
        assert_bits_equal(deq, O.mxint_quantizer(x, 32, 8), "packed: dequantized output")
        sc, mant = O.mxint_components(x.flatten(), 32, 8, 8)
        assert torch.equal(codes.cpu().view(-1, 32).float(), mant.float())
        assert torch.equal(scales.cpu().float().view(-1, 1), sc.float())
        rebuilt = codes.cpu().view(-1, 32).double() * torch.exp2(scales.cpu().double().view(-1, 1) - 134)
        assert torch.equal(rebuilt.view_as(x), deq.cpu().double())


# ------------------------------------------------------------------ block floating point
BFP_CASES = [
    ((2, 6, 64), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 16], skip_first_dim=True)),
    ((2, 5, 40), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[2, 16], skip_first_dim=True)),
    ((2, 4, 48), dict(width=6, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=True)),
    ((5, 50), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=True)),
    ((12, 40), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[4, 16], skip_first_dim=False)),
    ((7, 64), dict(width=12, exponent_width=8, exponent_bias=None, block_size=[1, 16], skip_first_dim=False)),
    ((33, 64), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=False)),
    ((37,), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=False)),
    ((64,), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=False)),
    ((2, 6, 64), dict(width=4, exponent_width=4, exponent_bias=None, block_size=[1, 16], skip_first_dim=True)),
    ((2, 6, 64), dict(width=12, exponent_width=5, exponent_bias=3, block_size=[1, 32], skip_first_dim=True)),
    ((3, 8, 256), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 4], skip_first_dim=True)),
    ((3, 8, 256), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 128], skip_first_dim=True)),
    ((3, 8, 512), dict(width=16, exponent_width=8, exponent_bias=None, block_size=[1, 512], skip_first_dim=True)),
    ((4, 96), dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 2], skip_first_dim=True)),
]


def bfp_input(rng, shape, dtype):
    n = int(np.prod(shape))
    x = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).to(dtype)
    flat = x.view(-1)
    flat[rng.integers(0, n, size=max(1, n // 16))] *= 50
    idx = rng.integers(0, n, size=max(1, n // 8))
    flat[idx] = torch.from_numpy((2.0 ** rng.integers(-6, 9, size=idx.size)).astype(np.float32)).to(dtype)
    idx = rng.integers(0, n, size=max(1, n // 16))
    flat[idx] = torch.from_numpy((1e-8 * rng.uniform(0.5, 2.0, size=idx.size)).astype(np.float32)).to(dtype)
    flat[rng.integers(0, n, size=max(1, n // 16))] = 0.0
    flat[rng.integers(0, n, size=max(1, n // 32))] = -0.0
    if n >= 32:
        flat[:16] = 0.0
    if dtype != torch.float32:
        idx = rng.integers(0, n, size=max(1, n // 16))
        p2 = torch.from_numpy((2.0 ** rng.integers(4, 9, size=idx.size)).astype(np.float32)).to(dtype)
        flat[idx] = (p2.view(torch.int16) + 1).view(dtype)
    return x.view(shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=_ID.get)
@pytest.mark.parametrize("case", range(len(BFP_CASES)))
def test_block_fp_cases(Q, dev, dtype, case):
    shape, kw = BFP_CASES[case]
    rng = np.random.default_rng(300 + case)
    x = bfp_input(rng, shape, dtype)
    want = O.block_fp_quantizer(x.clone(), **kw)
    got = Q.block_fp_quantizer(x.to(dev), **kw)
    assert_bits_equal(got, want, f"block_fp {dtype} {shape} {kw}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=_ID.get)
def test_block_fp_every_16bit_value(Q, dev, dtype):
    """Every finite value of the dtype, as a block maximum and as a small element next to a large one."""
    v = all_16bit(dtype)
    x = torch.zeros(65536, 16, dtype=dtype)
    x[:, 0] = v
    x[:, 1] = (v.float() * 0.37).to(dtype)
    x[:, 2] = (v.float() * -0.011).to(dtype)
    y = torch.zeros(65536, 16, dtype=dtype)
    y[:, 0] = 1.5
    y[:, 1] = v
    for t, nm in ((x, "as max"), (y, "beside 1.5")):
        kw = dict(width=8, exponent_width=8, exponent_bias=None, block_size=[16], skip_first_dim=True)
        if dtype == torch.float16 and nm == "beside 1.5":
            t = t.clone()
            t[:, 1] = torch.where(t[:, 1].float().abs() > 1.5, torch.zeros_like(t[:, 1]), t[:, 1])
        assert_bits_equal(Q.block_fp_quantizer(t.to(dev), **kw), O.block_fp_quantizer(t.clone(), **kw), f"bfp all {nm}")


def test_block_fp_errors(Q, dev):
    with pytest.raises(NotImplementedError):
        Q.block_fp_quantizer(torch.zeros(2, 3, 4, device=dev), 8, 8, None, [16], skip_first_dim=False)
    with pytest.raises(RuntimeError):
        Q.block_fp_quantizer(torch.zeros(2, 3, 4, 5, device=dev), 8, 8, None, [16], skip_first_dim=True)
    with pytest.raises(AssertionError):
        Q.block_fp_quantizer(torch.zeros(8, device=dev), 8, 8, None, [16], skip_first_dim=True)


# ------------------------------------------------------------------ fixed point
@pytest.mark.parametrize("width,frac,signed", [(8, 4, True), (8, 0, True), (4, 6, True), (8, -2, True), (8, 4, False),
                                               (16, 8, True), (2, 0, True), (12, None, True), (32, 16, True)])
def test_integer(Q, dev, width, frac, signed):
    rng = np.random.default_rng(width * 31 + (frac or 0))
    for dtype in DTYPES:
        if dtype == torch.float16 and width > 16:
            continue  # the clamp bound does not fit fp16: the reference raises there
        if dtype == torch.float32:
            x = fp32_from_bits(adversarial_fp32_bits(rng, 1 << 16))
            x = torch.where(torch.isfinite(x), x, torch.zeros_like(x))
            x = torch.cat([x, torch.randn(4099) * 8, (torch.arange(-2048, 2048).float() + 0.5) / 2 ** (frac or width // 2)])
        else:
            x = all_16bit(dtype)
        for fn in ("integer_quantizer", "integer_floor_quantizer"):
            want = getattr(O, fn)(x, width, frac, signed)
            got = getattr(Q, fn)(x.to(dev), width, frac, signed)
            assert_bits_equal(got, want, f"{fn} {dtype} w={width} f={frac} signed={signed}")


# ------------------------------------------------------------------ element-wise minifloat
@pytest.mark.parametrize("cfg", [(8, 4, None), (8, 5, None), (6, 3, None), (8, 4, 11), (12, 5, None), (16, 8, None),
                                 (8, 2, None), (4, 2, 0), (8, 5, 25), (8, 6, None), (6, 5, 31)])
@pytest.mark.parametrize("dtype", DTYPES, ids=_ID.get)
def test_minifloat_denorm_ieee(Q, dev, dtype, cfg):
    w, ew, eb = cfg
    rng = np.random.default_rng(w * 100 + ew)
    if dtype == torch.float32:
        x = fp32_from_bits(adversarial_fp32_bits(rng, 1 << 16))
        x = torch.where(torch.isfinite(x), x, torch.zeros_like(x))
        x = torch.cat([x, torch.randn(5001) * 3])
    else:
        x = all_16bit(dtype)
    for name in ("minifloat_denorm_quantizer", "minifloat_ieee_quantizer"):
        want = getattr(O, name)(x, w, ew, eb)
        got = getattr(Q, name)(x.to(dev), w, ew, eb)
        assert_bits_equal(got, want, f"{name} {dtype} {cfg}")


# ------------------------------------------------------------------ bit-level minifloat and MXFP
MF_FORMATS = [(4, 3), (5, 2), (2, 1), (2, 3), (3, 2), (1, 2), (5, 10), (8, 7), (3, 4), (5, 8), (4, 9), (8, 6)]


@pytest.mark.parametrize("fmt", MF_FORMATS)
@pytest.mark.parametrize("finite", [True, False])
def test_minifloat_mx(Q, dev, fmt, finite):
    e, f = fmt
    rng = np.random.default_rng(e * 16 + f)
    xf = fp32_from_bits(np.concatenate([adversarial_fp32_bits(rng, 1 << 16), np.arange(65536, dtype=np.uint32) << 16]))
    if finite:
        xf = torch.where(torch.isfinite(xf), xf, torch.zeros_like(xf))
    for rm in ("rn", "ru", "rd", "rz"):
        meta = Q.MinifloatMeta(e, f, finite, rm)
        want = O.minifloat_quantizer_sim(xf, e, f, finite, rm)
        got = Q.minifloat_quantizer_sim(xf.to(dev), meta)
        assert_bits_equal(got, want, f"minifloat_mx e{e}m{f} finite={finite} {rm}")
    for dtype in (torch.bfloat16, torch.float16):
        x = all_16bit(dtype)
        for rm in ("rn", "ru", "rd", "rz"):  # every 16-bit value in every mode: the packed 16-bit kernel's domain
            meta = Q.MinifloatMeta(e, f, finite, rm)
            assert_bits_equal(Q.minifloat_quantizer_sim(x.to(dev), meta), O.minifloat_quantizer_sim(x, e, f, finite, rm),
                              f"minifloat_mx {dtype} e{e}m{f} finite={finite} {rm}")
            # a lane's 8 elements are handled together: shuffled order and an unaligned view
            perm = torch.randperm(65536, generator=torch.Generator().manual_seed(e * 8 + f))
            xs = x[perm]
            assert_bits_equal(Q.minifloat_quantizer_sim(xs.to(dev)[3:], meta), O.minifloat_quantizer_sim(xs[3:], e, f, finite, rm),
                              f"minifloat_mx {dtype} e{e}m{f} {rm} shuffled")
        meta = Q.MinifloatMeta(e, f, finite, "rn")
        assert_bits_equal(Q.minifloat_quantizer_sim(x.to(dev), meta, output_dtype=torch.float32),
                          O.minifloat_quantizer_sim(x, e, f, finite, "rn", torch.float32), "output dtype")


@pytest.mark.parametrize("fmt", [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2)])
@pytest.mark.parametrize("dtype", DTYPES, ids=_ID.get)
def test_mxfp(Q, dev, dtype, fmt):
    e, f = fmt
    rng = np.random.default_rng(e * 8 + f)
    for B in (32, 16, 8, 4, 64, 24):
        x = adversarial(rng, (48, 768), dtype, block=B if 768 % B == 0 else 8)
        want = O.mxfp_quantizer(x, B, e, f)
        got = Q.mxfp_quantizer(x.to(dev), B, e, f)
        assert_bits_equal(got, want, f"mxfp {dtype} e{e}m{f} B={B}")
    x = adversarial(rng, (6, 64, 40), dtype, block=8)
    for dim, B in [(1, 32), (0, 2), (-1, 8)]:
        assert_bits_equal(Q.mxfp_quantizer(x.to(dev), B, e, f, block_dim=dim), O.mxfp_quantizer(x, B, e, f, block_dim=dim),
                          f"mxfp dim={dim}")


@pytest.mark.parametrize("fmt", [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=_ID.get)
def test_mxfp_every_16bit_value_as_an_element(Q, dev, dtype, fmt):
    """every finite 16-bit pattern as an element of blocks whose maximum sits 0 .. 100 binades above it (the packed
    16-bit kernel: ordinary codes, the format's subnormal binade, underflow, quotients that leave the fp32 range)"""
    e, f = fmt
    x = all_16bit(dtype)
    x = x[torch.isfinite(x)]
    x = x[: (x.numel() // 31) * 31].view(-1, 31)
    top = float(torch.finfo(dtype).max)
    for lift in (0, 1, 2, 3, 6, 9, 16, 40, 100):
        mx = (x.double().abs().max(dim=1, keepdim=True).values * 2.0 ** lift).clamp(max=top / 2).to(dtype)
        blocks = torch.cat([x, mx], dim=1).contiguous()
        assert_bits_equal(Q.mxfp_quantizer(blocks.to(dev), 32, e, f), O.mxfp_quantizer(blocks, 32, e, f),
                          f"mxfp {dtype} e{e}m{f} lift {lift}")
    g = torch.Generator().manual_seed(e * 8 + f)
    shuffled = all_16bit(dtype)
    shuffled = shuffled[torch.isfinite(shuffled)]
    shuffled = shuffled[torch.randperm(shuffled.numel(), generator=g)][: (shuffled.numel() // 64) * 64].view(-1, 64)
    for B in (8, 16, 32, 64):
        assert_bits_equal(Q.mxfp_quantizer(shuffled.to(dev), B, e, f), O.mxfp_quantizer(shuffled, B, e, f),
                          f"mxfp {dtype} e{e}m{f} shuffled B={B}")


def test_mxfp_top_of_range_and_subnormals(Q, dev):
    """Scaled values in [448, 512) (the all-finite e4m3 top codes and the lost-carry binade) and fp32 subnormals."""
    top = torch.tensor([464, 479.9, 480, 495.9, 496, 511.9, 448, 300, 1.9375 * 128, 1.97 * 64, 1.97 * 32], dtype=torch.float32)
    rows = []
    for s in (-20, -3, 0, 7):
        r = torch.full((32,), 0.01 * 2.0 ** s)
        r[: top.numel()] = top / 256 * 2.0 ** s
        rows.append(r)
        rows.append(-r)
    sub = torch.arange(1, 33, dtype=torch.int32).view(torch.float32)
    rows.append(sub)
    mixed = sub.clone()
    mixed[4] = 1.0e-30
    rows.append(mixed)
    x = torch.stack(rows)
    for (e, f) in [(4, 3), (5, 2), (2, 1)]:
        assert_bits_equal(Q.mxfp_quantizer(x.to(dev), 32, e, f), O.mxfp_quantizer(x, 32, e, f), f"mxfp top e{e}m{f}")


def test_mxfp_illegal_format(Q, dev):
    with pytest.raises(AssertionError):
        Q.mxfp_quantizer(torch.zeros(4, 32, device=dev), 32, 3, 3)


# ------------------------------------------------------------------ autograd and device contract
def test_straight_through_gradient(Q, dev):
    x = torch.randn(8, 64, device=dev, requires_grad=True)
    for fn in (lambda t: Q.mxint_quantizer(t, 32, 8), lambda t: Q.block_fp_quantizer(t, 8, 8, None, [16]),
               lambda t: Q.integer_quantizer(t, 8, 4), lambda t: Q.mxfp_quantizer(t, 32, 4, 3),
               lambda t: Q.minifloat_ieee_quantizer(t, 8, 4)):
        x.grad = None
        g = torch.randn(8, 64, device=dev)
        fn(x).backward(g)
        assert torch.equal(x.grad, g)


def test_cpu_tensor_is_rejected(Q):
    from mase_amd._lib import MaseAmdError

    with pytest.raises(MaseAmdError):
        Q.mxint_quantizer(torch.randn(4, 32), 32, 8)
