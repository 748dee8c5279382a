"""GPU tests of the packed-MXFP path: the packer against the oracle quantizer, and the block-scaled MFMA
contraction against an fp64 product of the decoded operands."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import adversarial

pytestmark = pytest.mark.gpu


def decode_ocp(codes: torch.Tensor, scales: torch.Tensor, fmt):
    """packed hardware codes + E8M0 scales -> float64 values, decoded per the OCP MX formats"""
    E, F = fmt
    c = codes.cpu().to(torch.int64)
    if E + F + 1 <= 4:
        c = torch.stack([c & 0xF, c >> 4], dim=-1).reshape(*c.shape[:-1], -1)
    bias = (1 << (E - 1)) - 1
    sgn = (c >> (E + F)) & 1
    e = (c >> F) & ((1 << E) - 1)
    f = c & ((1 << F) - 1)
    mag = torch.where(e == 0, f.double() / (1 << F) * 2.0 ** (1 - bias), (1 + f.double() / (1 << F)) * torch.exp2((e - bias).double()))
    if (E, F) == (4, 3):
        assert not bool(((e == 15) & (f == 7)).any()), "packed e4m3 must not contain the NaN code"
    if (E, F) == (5, 2):
        assert not bool((e == 31).any()), "packed e5m2 must not contain Inf/NaN codes"
    v = torch.where(sgn == 1, -mag, mag)
    s = torch.exp2(scales.cpu().double() - 127).repeat_interleave(32, dim=-1)
    return v * s


@pytest.mark.parametrize("fmt", [(4, 3), (5, 2), (2, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mxfp_pack_decodes_to_the_quantizer_output(dev, fmt, dtype):
    from mase_amd._gemm import mxfp_pack

    rng = np.random.default_rng(fmt[0] * 4 + fmt[1])
    x = adversarial(rng, (64, 512), dtype, block=32)
    x = torch.where(x.float().abs() < 1e20, x, torch.zeros_like(x))
    x[3, :32] = torch.linspace(-1, 1, 32).to(dtype) * 479.0 / 256  # a block whose maximum rounds to the top e4m3 code
    want = O.mxfp_quantizer(x.float(), 32, fmt[0], fmt[1]).double()
    codes, scales = mxfp_pack(x.to(dev), *fmt)
    got = decode_ocp(codes, scales, fmt)
    blk_max = want.abs().reshape(64, -1, 32).amax(-1, keepdim=True).repeat_interleave(32, -1).reshape(64, 512)
    diff = (got - want).abs()
    # exact except in blocks re-expressed with the next scale, where elements far below the block maximum
    # are rounded into the format's subnormal range
    assert float((diff / blk_max.clamp_min(1e-300)).max()) <= 2.0 ** -9
    exact = float((diff == 0).double().mean())
    print(f"pack e{fmt[0]}m{fmt[1]} {dtype}: {exact:.4f} of elements exact")
    assert exact > (0.97 if fmt != (5, 2) else 0.5)
    assert bool(((got == 0) == (want == 0)).all()) or fmt == (5, 2)


@pytest.mark.parametrize("fmt", [(4, 3), (5, 2)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mxfp_pack_of_16bit_tensors_is_the_fp32_packing_of_the_same_values(dev, fmt, dtype):
    """16-bit tensors take the kernel that derives the codes from the packed 16-bit cast; fp32 tensors the one that
    encodes on the fp32 bit fields.  Same values in, same codes and scale bytes out: adversarial values (powers of two
    and their neighbours, zeros, subnormals of the dtype, huge spreads inside a block), plain normal data, blocks that
    use the reserved codes and a block of non-finite values."""
    from mase_amd._gemm import mxfp_pack, mxfp_pack_tiled, mxfp_tile_codes

    rng = np.random.default_rng(100 + fmt[0])
    g = torch.Generator().manual_seed(7)
    parts = [adversarial(rng, (96, 512), dtype, block=32), torch.randn(700, 512, generator=g).to(dtype),
             (torch.randn(64, 512, generator=g) * torch.exp2(torch.randint(-20, 12, (64, 512), generator=g).float())).to(dtype)]
    x = torch.cat(parts)
    x[5, :32] = torch.linspace(-1, 1, 32).to(dtype) * 479.0 / 256   # maximum on the top e4m3 code
    x[6, 32:64] = torch.linspace(-1, 1, 32).to(dtype) * 7.5          # and one that rounds up to it
    x[7, :32] = float("inf")
    x[8, 64:96] = float("nan")
    x[9, :64] = 0
    x[10, :32] = torch.tensor(2.0 ** -14 if dtype == torch.float16 else 2.0 ** -120).to(dtype) / 3  # subnormal / tiny
    xd = x.to(dev)
    c16, s16 = mxfp_pack(xd, *fmt)
    c32, s32 = mxfp_pack(xd.float(), *fmt)
    assert torch.equal(s16, s32)
    bad = (c16 != c32)
    assert not bool(bad.any()), (int(bad.sum()), x[bad.cpu()][:8], c16[bad][:8], c32[bad][:8])
    for rows, K in ((3, 96), (1, 32), (5, 160), (7, 128)):  # block counts that are and are not multiples of 4
        xs = xd[:rows, :K].contiguous()
        a, b = mxfp_pack(xs, *fmt)
        c, d = mxfp_pack(xs.float(), *fmt)
        assert torch.equal(a, c) and torch.equal(b, d), (rows, K)
    t16, ts16 = mxfp_pack_tiled(xd, *fmt)
    assert torch.equal(ts16, s32)
    want = mxfp_tile_codes(c32, 512, 8).cpu().reshape(-1, 4, 256, 128).permute(0, 2, 1, 3)
    got = t16.cpu().reshape(-1, 4, 256, 128).permute(0, 2, 1, 3)
    live = torch.arange(want.shape[0] * 256).reshape(-1, 256) < x.shape[0]  # padding rows are left unwritten
    assert torch.equal(got[live], want[live])


@pytest.mark.parametrize("bfmt", [(2, 1), (4, 3), (5, 2)])
@pytest.mark.parametrize("afmt", [(4, 3), (5, 2)])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 384), (512, 768, 1024), (1, 33, 256)])
def test_gemm_mxfp_scaled_against_decoded_operands(dev, afmt, bfmt, M, N, K):
    from mase_amd._gemm import gemm_mxfp_scaled, mxfp_pack

    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g)
    a[:, 5] *= 20
    b = torch.randn(N, K, generator=g) * 0.02
    bias = torch.randn(N, generator=g)
    print(f"mxfp gemm {afmt}x{bfmt} M={M} N={N} K={K}", flush=True)
    ac, asc = mxfp_pack(a.to(dev), *afmt)
    bc, bsc = mxfp_pack(b.to(dev), *bfmt)
    da, db = decode_ocp(ac, asc, afmt), decode_ocp(bc, bsc, bfmt)
    ref = da @ db.t()
    # The instruction adds the 8 products of one register pair after aligning them to the largest of the 8
    # and dropping what lies more than about 12 bits below its leading bit (measured: e4m3 x e2m1 keeps a
    # granularity of 2^-12 of that product); sums across such groups and across instructions are fp32.
    # Hence |error| <= 7 * 2^-12 * sum|a_k b_k| in the worst case; typical errors are ~1e-5 of the result.
    bound = (da.abs() @ db.abs().t()) * 2.0 ** -9 + ref.abs() * 2.0 ** -21
    y = gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, bfmt, None, torch.float32)
    d = (y.cpu().double() - ref).abs()
    assert bool((d <= bound).all()), float((d / bound).max())
    err = float(d.max() / ref.abs().max())
    print(f"  max |err| / max |ref| = {err:.2e}")
    assert err < 5e-4, err
    yb = gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, bfmt, bias.to(dev), torch.bfloat16)
    want = ref + bias.double()
    d = (yb.cpu().double() - want).abs()
    assert bool((d <= want.abs() * 2.0 ** -8 + ref.abs().max() * 5e-4).all())  # bf16 rounding of the output
    # the epilogue's forms agree bit for bit: a 16-bit output is the fp32 output rounded once, with or without a bias
    # (which is added in fp32 before the rounding)
    for dt in (torch.bfloat16, torch.float16):
        assert torch.equal(gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, bfmt, None, dt), y.to(dt)), dt
    yf = gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, bfmt, bias.to(dev), torch.float32)
    assert torch.equal(yf, y + bias.to(dev))
    assert torch.equal(yb, yf.to(torch.bfloat16))
    assert torch.equal(gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, bfmt, bias.to(dev).half(), torch.float16),
                       (y + bias.to(dev).half().float()).half())


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gemm_mxfp_output_not_on_a_16_byte_boundary(dev, dt, with_bias):
    """the epilogue's element-by-element stores on full tiles: C handed over 4 bytes past a 16-byte boundary (the C ABI
    asks for no alignment of C), the same values as in an aligned C and nothing written outside it"""
    from mase_amd import _lib
    from mase_amd._gemm import MXFP_HW_FORMATS, gemm_mxfp_scaled, mxfp_pack

    lib = _lib.load()
    M, N, K = 512, 520, 256
    g = torch.Generator().manual_seed(11)
    ac, asc = mxfp_pack(torch.randn(M, K, generator=g).to(dev), 4, 3)
    bc, bsc = mxfp_pack((torch.randn(N, K, generator=g) * 0.02).to(dev), 2, 1)
    bias = torch.randn(N, generator=g).to(dev) if with_bias else None
    want = gemm_mxfp_scaled(ac, asc, (4, 3), bc, bsc, (2, 1), bias, dt)
    shift = 4 // want.element_size()
    buf = torch.zeros(M * N + 16, dtype=dt, device=dev)
    c = buf[shift: shift + M * N]
    assert c.data_ptr() % 16 == 4
    rc = lib.mase_gemm_mxfp_scaled(ac.data_ptr(), asc.data_ptr(), MXFP_HW_FORMATS[(4, 3)], bc.data_ptr(), bsc.data_ptr(),
                                   MXFP_HW_FORMATS[(2, 1)], bias.data_ptr() if with_bias else None, c.data_ptr(), M, N, K,
                                   _lib.DTYPE_CODE[dt], 0, _lib.stream_ptr(ac))
    assert rc == 0
    assert torch.equal(c.view(M, N), want)
    assert float(buf[:shift].abs().max()) == 0 and float(buf[shift + M * N:].abs().max()) == 0


def test_gemm_mxfp_exact_small_integers(dev):
    """e2m1 x e4m3 with unit scales and values that both formats hold exactly: every product is a multiple of 32
    below 2^11, so neither the 12-bit alignment inside the instruction nor fp32 accumulation rounds anything"""
    from mase_amd._gemm import gemm_mxfp_scaled, mxfp_pack

    g = torch.Generator().manual_seed(1)
    a = torch.randint(-8, 9, (256, 256), generator=g).float() * 32   # multiples of 32 up to 256: exact in e4m3
    a[:, ::32] = 256.0  # pins every block's scale
    b = torch.tensor([0, 1, 1.5, 2, 3, 4, 6, 6])[torch.randint(0, 8, (256, 256), generator=g)] * torch.where(torch.rand(256, 256, generator=g) < 0.5, -1.0, 1.0)
    b[:, ::32] = 6.0
    ac, asc = mxfp_pack(a.to(dev), 4, 3)
    bc, bsc = mxfp_pack(b.to(dev), 2, 1)
    assert torch.equal(decode_ocp(ac, asc, (4, 3)), a.double()) and torch.equal(decode_ocp(bc, bsc, (2, 1)), b.double())
    y = gemm_mxfp_scaled(ac, asc, (4, 3), bc, bsc, (2, 1), None, torch.float32)
    assert torch.equal(y.cpu().double(), a.double() @ b.double().t())


@pytest.mark.parametrize("bfmt", [(2, 1), (4, 3)])
@pytest.mark.parametrize("M,N,K", [(4096, 8192, 384), (4352, 4352, 256), (2048, 8448, 128), (4100, 4200, 640)])
def test_gemm_mxfp_several_tiles_per_work_group(dev, bfmt, M, N, K):
    """more output tiles than CUs (the K-tile stream of a work-group crosses from one output tile to the next), with
    K of 1 to 5 tiles; operands chosen so that every product and partial sum is exact: bit-exact result required"""
    from mase_amd._gemm import gemm_mxfp_scaled, mxfp_pack

    g = torch.Generator().manual_seed(M + N + K + bfmt[0])
    a = torch.randint(-8, 9, (M, K), generator=g).float() * 32
    a[:, ::32] = 256.0  # pins every block's scale
    vals = torch.tensor([0, 1, 1.5, 2, 3, 4, 6, 6]) if bfmt == (2, 1) else torch.tensor([0, 32, 64, 96, 128, 160, 192, 224.0])
    top = 6.0 if bfmt == (2, 1) else 256.0
    b = vals[torch.randint(0, 8, (N, K), generator=g)] * torch.where(torch.rand(N, K, generator=g) < 0.5, -1.0, 1.0)
    b[:, ::32] = top
    print(f"mxfp gemm multi-tile {bfmt} M={M} N={N} K={K}", flush=True)
    ad, bd = a.to(dev), b.to(dev)
    ac, asc = mxfp_pack(ad, 4, 3)
    bc, bsc = mxfp_pack(bd, *bfmt)
    ref = (ad @ bd.t()).cpu()  # exact in fp32: multiples of 32 (or 1024) well below 2^24 units
    y = gemm_mxfp_scaled(ac, asc, (4, 3), bc, bsc, bfmt, None, torch.float32)
    assert torch.equal(y.cpu(), ref)


@pytest.mark.parametrize("afmt", [(4, 3), (5, 2)])
@pytest.mark.parametrize("M", [1, 9, 16, 32, 33, 100, 128])
def test_gemm_mxfp4_few_rows_streams_the_weight_codes(dev, afmt, M):
    """mase_gemm_mxfp4_skinny against the decoded operands (same bound as the tiled kernel: the instruction is the
    same) and against the tiled kernel itself; reproducible; bias and output dtypes"""
    from mase_amd._gemm import gemm_mxfp4_skinny, gemm_mxfp_scaled, mxfp_pack

    g = torch.Generator().manual_seed(M * 7 + afmt[0])
    for (N, K) in [(64, 128), (4096, 4096), (1000, 1152), (11008, 2048), (512, 7936), (4096, 11008)]:  # 31, 43 chunks: unequal K ranges
        a = torch.randn(M, K, generator=g)
        a[:, 5] *= 20
        b = torch.randn(N, K, generator=g) * 0.02
        b[3] *= 2.0 ** -30
        b[5, :64] = 0.0
        bias = torch.randn(N, generator=g)
        ac, asc = mxfp_pack(a.to(dev), *afmt)
        bc, bsc = mxfp_pack(b.to(dev), 2, 1)
        da, db = decode_ocp(ac, asc, afmt), decode_ocp(bc, bsc, (2, 1))
        ref = da @ db.t()
        bound = (da.abs() @ db.abs().t()) * 2.0 ** -9 + ref.abs() * 2.0 ** -21
        y = gemm_mxfp4_skinny(ac, asc, afmt, bc, bsc, None, torch.float32)
        d = (y.cpu().double() - ref).abs()
        assert bool((d <= bound).all()), (N, K, float((d / bound).max()))
        assert float(d.max() / ref.abs().max()) < 5e-4
        tiled = gemm_mxfp_scaled(ac, asc, afmt, bc, bsc, (2, 1), None, torch.float32)
        assert float((y - tiled).abs().max() / ref.abs().max()) < 5e-4
        assert torch.equal(y, gemm_mxfp4_skinny(ac, asc, afmt, bc, bsc, None, torch.float32))
        yb = gemm_mxfp4_skinny(ac, asc, afmt, bc, bsc, bias.to(dev), torch.bfloat16)
        want = ref + bias.double()
        assert bool(((yb.cpu().double() - want).abs() <= want.abs() * 2.0 ** -8 + ref.abs().max() * 5e-4).all())
    # exact case: unit scales, small integers both formats hold exactly
    N, K = 96, 256
    ai = torch.randint(-4, 5, (M, K), generator=g).float()
    bi = torch.randint(-3, 4, (N, K), generator=g).float()
    ai[:, 0], bi[:, 0] = 4.0, 3.0
    ac, asc = mxfp_pack(ai.to(dev), *afmt)
    bc, bsc = mxfp_pack(bi.to(dev), 2, 1)
    da, db = decode_ocp(ac, asc, afmt), decode_ocp(bc, bsc, (2, 1))
    if torch.equal(da.float(), ai) and torch.equal(db.float(), bi):
        assert torch.equal(gemm_mxfp4_skinny(ac, asc, afmt, bc, bsc, None, torch.float32).cpu().double(), da @ db.t())


def tile_image(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """The tile image of a row-major code matrix, spelled out with indices: [row tile of 256][K tile of 128][row]
    [128 or 64 bytes], 16-byte chunk c of a row segment at position c ^ swizzle(row), rows past the end repeating the last."""
    codes = codes.cpu()
    rows, row_bytes = codes.shape
    seg = 128 * bits // 8
    nk = row_bytes // seg
    tiles = -(-rows // 256)
    r = torch.arange(tiles * 256).clamp(max=rows - 1)
    src = codes[r].reshape(tiles, 256, nk, seg // 16, 16)
    rr = torch.arange(256)
    sw = ((rr >> 1) & 7) if bits == 8 else ((rr >> 2) & 3)
    pos = torch.arange(seg // 16)[None, :] ^ sw[:, None]              # [256, chunks]: position -> source chunk
    img = src[:, rr[:, None], :, pos, :]                                # [256, chunks, tiles, nk, 16]
    return img.permute(2, 3, 0, 1, 4).reshape(-1).contiguous()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("rows,K", [(256, 128), (300, 384), (1, 256), (777, 1024)])
def test_mxfp_tile_codes_is_the_stated_permutation(dev, bits, rows, K):
    from mase_amd._gemm import mxfp_tile_codes

    g = torch.Generator().manual_seed(rows + K + bits)
    codes = torch.randint(0, 256, (rows, K * bits // 8), generator=g, dtype=torch.uint8)
    got = mxfp_tile_codes(codes.to(dev), K, bits).cpu()
    assert torch.equal(got, tile_image(codes, bits))


@pytest.mark.parametrize("fmt", [(4, 3), (5, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,K", [(256, 128), (300, 384), (3, 1024)])
def test_mxfp_pack_tiled_writes_the_image_of_the_row_major_codes(dev, fmt, dtype, rows, K):
    from mase_amd._gemm import mxfp_pack, mxfp_pack_tiled

    rng = np.random.default_rng(rows + K)
    x = adversarial(rng, (rows, K), dtype, block=32)
    x = torch.where(x.float().abs() < 1e4, x, torch.zeros_like(x)).to(dev)
    codes, scales = mxfp_pack(x, *fmt)
    tiled, tscales = mxfp_pack_tiled(x, *fmt)
    assert torch.equal(scales, tscales)
    want = tile_image(codes, 8).reshape(-1, K // 128, 256, 128)
    got = tiled.cpu().reshape(-1, K // 128, 256, 128)
    live = torch.arange(want.shape[0] * 256).reshape(-1, 256) < rows   # padding rows are left unwritten
    assert torch.equal(got.permute(0, 2, 1, 3)[live], want.permute(0, 2, 1, 3)[live])


@pytest.mark.parametrize("afmt", [(4, 3), (5, 2)])
@pytest.mark.parametrize("out_dtype,with_bias", [(torch.bfloat16, False), (torch.float32, True), (torch.float16, True)])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 384), (512, 768, 1024), (129, 33, 256), (1024, 512, 2048)])
def test_gemm_mxfp4_on_tile_images_is_the_same_product(dev, afmt, out_dtype, with_bias, M, N, K):
    from mase_amd._gemm import gemm_mxfp4_scaled_tiled, gemm_mxfp_scaled, mxfp_pack, mxfp_pack_tiled, mxfp_tile_codes

    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bias = torch.randn(N, generator=g).to(out_dtype).to(dev) if with_bias else None
    xc, xs = mxfp_pack(x, *afmt)
    wc, ws = mxfp_pack(w, 2, 1)
    want = gemm_mxfp_scaled(xc, xs, afmt, wc, ws, (2, 1), bias, out_dtype)
    xt, xts = mxfp_pack_tiled(x, *afmt)
    got = gemm_mxfp4_scaled_tiled(xt, xts, afmt, mxfp_tile_codes(wc, K, 4), ws, bias, out_dtype)
    assert torch.equal(got, want)
    # the activation image made from the row-major codes gives the same product as the one the quantizer writes
    got2 = gemm_mxfp4_scaled_tiled(mxfp_tile_codes(xc, K, 8), xs, afmt, mxfp_tile_codes(wc, K, 4), ws, bias, out_dtype)
    assert torch.equal(got2, want)
