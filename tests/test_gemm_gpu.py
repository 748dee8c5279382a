"""GPU parity of the bf16 matrix-core contraction against an fp32 reference of the same operands."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def rel_err(y, ref):
    """max |y - ref| / max |ref|: the error measure used for every Linear comparison in this repo"""
    return float((y.double() - ref.double()).abs().max() / ref.double().abs().max())


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (256, 256, 32), (512, 768, 128), (300, 200, 96), (1, 256, 64), (257, 513, 32),
                                   (1024, 1024, 1024), (4096, 4096, 4096), (130, 11008, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_tn(dev, M, N, K, out_dtype):
    from mase_amd._gemm import gemm_bf16_tn

    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    a = torch.randn(M, K, generator=g).bfloat16()
    b = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    bias = torch.randn(N, generator=g)
    print(f"gemm case M={M} N={N} K={K} out={out_dtype}", flush=True)
    ad, bd = a.to(dev), b.to(dev)
    ref = (ad.float() @ bd.float().t()).double().cpu() if M * N * K > 2 ** 28 else a.double() @ b.double().t()
    y = gemm_bf16_tn(ad, bd, None, out_dtype)
    tol = 2e-6 if out_dtype == torch.float32 else 4e-3  # fp32: summation order only; bf16: output rounding
    if M * N * K > 2 ** 28:
        tol = max(tol, 2e-5)  # the fp32 device reference itself carries rounding error at this size
    assert rel_err(y.cpu(), ref) < tol
    yb = gemm_bf16_tn(ad, bd, bias.to(dev), out_dtype)
    assert rel_err(yb.cpu(), ref + bias.double()) < tol
    yb2 = gemm_bf16_tn(ad, bd, bias.bfloat16().to(dev), out_dtype)
    assert rel_err(yb2.cpu(), ref + bias.bfloat16().double()) < tol


@pytest.mark.parametrize("M,N,K", [(4096, 8192, 192), (4352, 4352, 128), (2048, 8448, 64), (4100, 4200, 320)])
def test_gemm_bf16_tn_several_tiles_per_work_group(dev, M, N, K):
    """more 256x256 output tiles than CUs: every work-group walks several tiles and its K-tile stream crosses from
    one output tile to the next (tile counts divisible by 8 and not, K of 1, 2, 3 and 5 tiles).  Small-integer
    operands make every partial sum exact, so the result must equal the integer product bit for bit."""
    from mase_amd._gemm import gemm_bf16_tn

    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-16, 17, (M, K), generator=g).float()
    b = torch.randint(-16, 17, (N, K), generator=g).float()
    bias = torch.randint(-8, 9, (N,), generator=g).float()
    print(f"gemm multi-tile M={M} N={N} K={K}", flush=True)
    ad, bd = a.bfloat16().to(dev), b.bfloat16().to(dev)
    ref = (ad.float() @ bd.float().t()).cpu()   # exact in fp32 as well: |sums| < 2^24
    assert torch.equal(gemm_bf16_tn(ad, bd, None, torch.float32).cpu(), ref)
    assert torch.equal(gemm_bf16_tn(ad, bd, bias.to(dev), torch.float32).cpu(), ref + bias)
    yb = gemm_bf16_tn(ad, bd, None, torch.bfloat16).cpu()
    assert torch.equal(yb, ref.bfloat16())


def test_gemm_exact_on_small_integers(dev):
    """integer-valued operands with small K: every product and partial sum is exact in fp32, so the result
    must equal the integer matrix product bit for bit whatever the summation order"""
    from mase_amd._gemm import gemm_bf16_tn

    g = torch.Generator().manual_seed(5)
    a = torch.randint(-128, 128, (384, 256), generator=g).float()
    b = torch.randint(-128, 128, (320, 256), generator=g).float()
    y = gemm_bf16_tn(a.bfloat16().to(dev), b.bfloat16().to(dev), None, torch.float32)
    assert torch.equal(y.cpu(), a @ b.t())


def test_gemm_c_abi_rejects_partial_k_tiles(dev):
    from mase_amd import _lib

    lib = _lib.load()
    a = torch.zeros(4, 96, device=dev).bfloat16()
    c = torch.zeros(4, 4, device=dev)
    rc = lib.mase_gemm_bf16_tn(a.data_ptr(), a.data_ptr(), None, c.data_ptr(), 4, 4, 96, 0, 0, None)
    assert rc == -2


def test_gemm_wrappers_split_oversized_activations(dev, monkeypatch):
    """operands beyond the per-call size limit of the C entry points are fed in row chunks (limit lowered here so
    that a small problem exercises the split)"""
    from mase_amd import _gemm

    g = torch.Generator().manual_seed(3)
    a = torch.randint(-8, 9, (1000, 128), generator=g).float()
    b = torch.randint(-8, 9, (320, 128), generator=g).float()
    ad, bd = a.bfloat16().to(dev), b.bfloat16().to(dev)
    whole = _gemm.gemm_bf16_tn(ad, bd, None, torch.float32)
    monkeypatch.setattr(_gemm, "OPERAND_BYTES_LIMIT", 2 * 128 * 300)   # -> 256 rows per call
    assert torch.equal(_gemm.gemm_bf16_tn(ad, bd, None, torch.float32), whole)
    assert torch.equal(whole.cpu(), a @ b.t())
    monkeypatch.setattr(_gemm, "OPERAND_BYTES_LIMIT", (1 << 32) - 1)
    ac, asc = _gemm.mxfp_pack((a * 32).to(dev), 4, 3)
    bc, bsc = _gemm.mxfp_pack(b.to(dev), 4, 3)
    whole = _gemm.gemm_mxfp_scaled(ac, asc, (4, 3), bc, bsc, (4, 3), None, torch.float32)
    monkeypatch.setattr(_gemm, "OPERAND_BYTES_LIMIT", 128 * 300)
    assert torch.equal(_gemm.gemm_mxfp_scaled(ac, asc, (4, 3), bc, bsc, (4, 3), None, torch.float32), whole)


@pytest.mark.parametrize("M", [1, 7, 32, 33, 64, 100, 128])
@pytest.mark.parametrize("N,K", [(33, 64), (256, 4096), (4100, 1024), (11008, 4096), (4096, 11008), (520, 2368), (2048, 5504)])
def test_gemm_few_rows_takes_the_weight_streaming_kernel(dev, M, N, K):
    """M <= 128: the kernel that splits N and K over the chip and adds the K ranges in a fixed order.  Exact on
    small-integer operands, within fp32 summation error on random ones, and reproducible run to run.  K = 2368 and
    5504 are 37 and 86 chunks: no equal cut into ranges exists, the last range is shorter."""
    from mase_amd import _gemm

    assert M <= _gemm.SKINNY_MAX_ROWS
    g = torch.Generator().manual_seed(M * 13 + N + K)
    a = torch.randint(-8, 9, (M, K), generator=g).float()
    b = torch.randint(-8, 9, (N, K), generator=g).float()
    bias = torch.randint(-8, 9, (N,), generator=g).float()
    ad, bd = a.bfloat16().to(dev), b.bfloat16().to(dev)
    ref = a.double() @ b.double().t()
    assert torch.equal(_gemm.gemm_bf16_tn(ad, bd, None, torch.float32).cpu().double(), ref)
    assert torch.equal(_gemm.gemm_bf16_tn(ad, bd, bias.to(dev), torch.float32).cpu().double(), ref + bias.double())
    assert torch.equal(_gemm.gemm_bf16_tn(ad, bd, bias.bfloat16().to(dev), torch.bfloat16).cpu(), (ref + bias.double()).float().bfloat16())
    ar = torch.randn(M, K, generator=g).bfloat16()
    br = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    y1 = _gemm.gemm_bf16_tn(ar.to(dev), br.to(dev), None, torch.float32)
    y2 = _gemm.gemm_bf16_tn(ar.to(dev), br.to(dev), None, torch.float32)
    assert torch.equal(y1, y2)
    assert rel_err(y1.cpu(), ar.double() @ br.double().t()) < 2e-6


@pytest.mark.parametrize("M", [1, 7, 16, 32, 33, 100, 128])
def test_gemm_few_rows_with_mxint8_coded_weights(dev, M):
    """mase_gemm_mxint8_skinny: the weight as int8 codes + scale bytes.  The codes are widened to exactly the bf16
    values of the dequantized weight, so the result must agree with the bf16 product to fp32 summation order, and be
    exact when every partial sum is."""
    from mase_amd._gemm import gemm_bf16_tn, gemm_mxint8_skinny
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(M)
    for (N, K) in [(256, 128), (4096, 4096), (1000, 1152), (11008, 4096), (300, 5504), (2048, 3968)]:  # 43, 31 chunks: unequal K ranges
        w = (torch.randn(N, K, generator=g) * 0.05)
        w[3] *= 2.0 ** -40            # a row of tiny blocks (small scale bytes)
        w[5, :64] = 0.0               # all-zero blocks
        deq, codes, scales = _ops.mxint_qdq(w.to(dev), 32, 8, 1, 8, pack=True, out_dtype=torch.bfloat16)
        codes, scales = codes.view(N, K), scales.view(N, K // 32)
        a = torch.randn(M, K, generator=g).bfloat16().to(dev)
        bias = torch.randn(N, generator=g).to(dev)
        want = gemm_bf16_tn(a, deq, bias, torch.float32)
        got = gemm_mxint8_skinny(a, codes, scales, bias, torch.float32)
        ref = a.double() @ deq.double().T + bias.double()
        scale = float(ref.abs().max())
        assert float((got.double() - ref).abs().max()) / scale < 2e-6, (N, K)
        assert float((got - want).abs().max()) / scale < 2e-6, (N, K)
        assert torch.equal(got, gemm_mxint8_skinny(a, codes, scales, bias, torch.float32))   # reproducible
        got16 = gemm_mxint8_skinny(a, codes, scales, None, torch.bfloat16)
        assert float((got16.double() - (ref - bias.double())).abs().max()) / scale < 1e-2
    # exact case: small integers times powers of two, every partial sum exact in fp32
    N, K = 512, 256
    wi = torch.randint(-7, 8, (N, K), generator=g).float() * 0.25   # below the block maximum that saturates
    ai = torch.randint(-4, 5, (M, K), generator=g).float()
    deq, codes, scales = _ops.mxint_qdq(wi.to(dev), 32, 8, 1, 8, pack=True, out_dtype=torch.bfloat16)
    assert torch.equal(deq.float().cpu(), wi)
    got = gemm_mxint8_skinny(ai.bfloat16().to(dev), codes.view(N, K), scales.view(N, K // 32), None, torch.float32)
    assert torch.equal(got.cpu(), ai @ wi.T)


@pytest.mark.parametrize("kind", ["bf16", "mxint8", "mxfp4"])
@pytest.mark.parametrize("M,N,K", [(16, 32768, 256), (5, 32766, 512), (40, 33001, 256)])
def test_gemm_few_rows_single_k_range_finishes_the_output_in_the_kernel(dev, kind, M, N, K):
    """Wide weights with a short K take one K range: no reduction kernel runs, the weight-streaming kernel adds the
    bias and converts itself.  For every output and bias dtype the result must be the fp32 result plus the bias,
    rounded once; N = 32766 and 33001 take the scalar stores, 40 rows two passes."""
    from mase_amd import _gemm, _lib
    from mase_amd.quantizers import _ops

    lib = _lib.load()
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dev)
    if kind == "bf16":
        wb = w.bfloat16()
        assert lib.mase_gemm_bf16_skinny_workspace_bytes(M, N, K) == M * N * 4   # one K range
        run = lambda bias, dt: _gemm.gemm_bf16_tn(a, wb, bias, dt)
    elif kind == "mxint8":
        _, codes, scales = _ops.mxint_qdq(w, 32, 8, 1, 8, pack=True, out_dtype=torch.bfloat16)
        codes, scales = codes.view(N, K), scales.view(N, K // 32)
        assert lib.mase_gemm_mxint8_skinny_workspace_bytes(M, N, K) == M * N * 4
        run = lambda bias, dt: _gemm.gemm_mxint8_skinny(a, codes, scales, bias, dt)
    else:
        ac, asc = _gemm.mxfp_pack(a, 4, 3)
        bc, bsc = _gemm.mxfp_pack(w, 2, 1)
        assert lib.mase_gemm_mxfp4_skinny_workspace_bytes(M, N, K) == M * N * 4
        run = lambda bias, dt: _gemm.gemm_mxfp4_skinny(ac, asc, (4, 3), bc, bsc, bias, dt)
    y32 = run(None, torch.float32)
    assert torch.isfinite(y32).all() and float(y32.abs().max()) > 0
    for bias_dt in (torch.float32, torch.bfloat16, torch.float16):
        bias = torch.randn(N, generator=g).to(bias_dt).to(dev)
        for out_dt in (torch.float32, torch.bfloat16, torch.float16):
            got = run(bias, out_dt)
            want = (y32 + bias.float()).to(out_dt)
            assert torch.equal(got.view(torch.int32 if out_dt == torch.float32 else torch.int16),
                               want.view(torch.int32 if out_dt == torch.float32 else torch.int16)), (bias_dt, out_dt)


@pytest.mark.parametrize("M", [129, 256, 300, 512, 1000])
def test_gemm_a_few_hundred_rows_cuts_k_into_work_items(dev, M):
    """mase_gemm_bf16_tn_splitk through the dispatch of gemm_bf16_tn: exact on integer operands, agrees with fp64
    otherwise, reproducible, bias and all output dtypes; a shape with enough tiles reports no workspace"""
    from mase_amd import _lib
    from mase_amd._gemm import gemm_bf16_tn

    lib = _lib.load()
    g = torch.Generator().manual_seed(M)
    for (N, K) in [(4096, 4096), (1024, 8192), (768, 1536), (11008, 4096)]:
        assert lib.mase_gemm_bf16_tn_splitk_workspace_bytes(M, N, K) % (M * N * 4) == 0
        ai = torch.randint(-3, 4, (M, K), generator=g).bfloat16().to(dev)
        bi = torch.randint(-3, 4, (N, K), generator=g).bfloat16().to(dev)
        bias = torch.randint(-5, 6, (N,), generator=g).float().to(dev)
        want = ai.double() @ bi.double().T + bias.double()
        for dt in (torch.float32, torch.bfloat16):
            got = gemm_bf16_tn(ai, bi, bias, dt)
            if dt == torch.float32:
                assert torch.equal(got.double(), want), (N, K)
            else:
                assert torch.equal(got, want.to(dt)), (N, K)
        a = torch.randn(M, K, generator=g).bfloat16().to(dev)
        b = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
        got = gemm_bf16_tn(a, b, None, torch.float32)
        ref = a.double() @ b.double().T
        assert float((got.double() - ref).abs().max() / ref.abs().max()) < 2e-6
        assert torch.equal(got, gemm_bf16_tn(a, b, None, torch.float32))
    assert lib.mase_gemm_bf16_tn_splitk_workspace_bytes(4096, 4096, 4096) == 0      # 256 tiles: nothing to split
    assert lib.mase_gemm_bf16_tn_splitk_workspace_bytes(512, 4096, 4096) > 0


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 768, 256), (300, 200, 384), (4096, 4096, 1024), (2048, 8448, 512),
                                   (4100, 4200, 640), (16384, 1024, 4096), (1000, 33, 128),
                                   (16384, 4096, 11008), (16384, 11008, 4096), (16131, 4096, 11008), (3000, 600, 11008)])
def test_gemm_with_the_weight_in_fragment_order_is_the_same_product(dev, M, N, K):
    """mase_gemm_bf16_tn_packed against mase_gemm_bf16_tn on the same operands: the same products added in the same
    order (both compute with the 16x16x32 matrix instruction, K step by K step), so bit-identical: (1) on small-integer
    operands, where every partial sum is exact in fp32 and the result is also the exact integer product; (2) on random
    operands (the bias and every output dtype), every launch.  One to several output tiles per work-group, ragged M and
    N, 1 to 86 pairs of K tiles (K = 11008 and N = 11008 at 16384 rows are the decoder layer's down / gate / up
    projections at batch 8 x seq 2048), and against an fp32 product."""
    from mase_amd._gemm import gemm_bf16_pack_b, gemm_bf16_packed_b_supported, gemm_bf16_tn

    g = torch.Generator().manual_seed(M + N + K)
    bias = torch.randn(N, generator=g).to(dev)
    print(f"packed-B gemm M={M} N={N} K={K}", flush=True)
    assert gemm_bf16_packed_b_supported(N, K) == (K % 128 == 0)
    big = M * N * K > (1 << 36)
    # (1) integers of magnitude <= 8 and <= 15: |sum| <= 120 * 11008 < 2^24
    a = torch.randint(-8, 9, (M, K), generator=g).to(torch.bfloat16).to(dev)
    b = torch.randint(-15, 16, (N, K), generator=g).to(torch.bfloat16).to(dev)
    bp = gemm_bf16_pack_b(b)
    assert bp.numel() == (N + 31) // 32 * 32 * K * 2
    for dt, bs in ((torch.float32, None), (torch.bfloat16, bias), (torch.float16, bias.to(torch.float16))):
        want = gemm_bf16_tn(a, b, bs, dt)
        # several launches: the kernel's loads are tracked by hand, and a mistake there shows up as a few wrong tiles
        # in some launches only
        for rep in range(4 if big else 2):
            got = gemm_bf16_tn(a, b, bs, dt, b_packed=bp)
            assert torch.equal(got, want), (dt, rep, float((got.float() - want.float()).abs().max()))
    if K % 128 == 0 and M * N <= (1 << 24):
        exact = (a.double() @ b.double().t()).float()   # every value an integer below 2^24
        assert torch.equal(gemm_bf16_tn(a, b, None, torch.float32, b_packed=bp), exact)
    # (2) random operands
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bp = gemm_bf16_pack_b(b)
    for dt, bs in ((torch.float32, None), (torch.bfloat16, bias), (torch.float16, bias.to(torch.float16))):
        want = gemm_bf16_tn(a, b, bs, dt)
        for rep in range(3 if big else 2):
            got = gemm_bf16_tn(a, b, bs, dt, b_packed=bp)
            assert torch.equal(got, want), (dt, rep, float((got.float() - want.float()).abs().max()))
    if K % 128 == 0 and M > 512:
        ref = (a.float() @ b.float().t())
        assert float((gemm_bf16_tn(a, b, None, torch.float32, b_packed=bp) - ref).abs().max() / ref.abs().max()) < 1e-5


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16])
def test_gemm_output_not_on_a_16_byte_boundary(dev, dt):
    """the epilogue's element-by-element stores on full tiles: C handed over 4 bytes past a 16-byte boundary (the C ABI
    asks for no alignment of C), the same values as in an aligned C"""
    from mase_amd import _lib
    from mase_amd._gemm import gemm_bf16_pack_b, gemm_bf16_tn

    lib = _lib.load()
    M, N, K = 512, 520, 256  # two tile columns in full and a ragged third; N a multiple of 8
    g = torch.Generator().manual_seed(7)
    # small integers: every partial sum is exact
    a = torch.randint(-8, 9, (M, K), generator=g).to(torch.bfloat16).to(dev)
    b = torch.randint(-15, 16, (N, K), generator=g).to(torch.bfloat16).to(dev)
    bias = torch.randn(N, generator=g).to(dev)
    bp = gemm_bf16_pack_b(b)
    want = gemm_bf16_tn(a, b, bias, dt, b_packed=bp)
    shift = 4 // want.element_size()
    buf = torch.zeros(M * N + 16, dtype=dt, device=dev)
    c = buf[shift: shift + M * N]
    assert c.data_ptr() % 16 == 4
    code = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[dt]
    for packed in (True, False):
        buf.zero_()
        if packed:
            rc = lib.mase_gemm_bf16_tn_packed(a.data_ptr(), bp.data_ptr(), bias.data_ptr(), c.data_ptr(), M, N, K, code, 0,
                                              _lib.stream_ptr(a))
        else:
            rc = lib.mase_gemm_bf16_tn(a.data_ptr(), b.data_ptr(), bias.data_ptr(), c.data_ptr(), M, N, K, code, 0,
                                       _lib.stream_ptr(a))
        assert rc == 0
        assert torch.equal(c.view(M, N), want), packed
        assert float(buf[:shift].abs().max()) == 0 and float(buf[shift + M * N:].abs().max()) == 0  # nothing outside C


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 768, 256), (300, 200, 384), (4096, 4096, 1024), (130, 4096, 512),
                                   (4100, 4200, 640), (16384, 1024, 4096), (16384, 4096, 11008), (16131, 11008, 4096)])
def test_gemm_with_the_weight_as_mxint8_codes_in_fragment_order(dev, M, N, K):
    """mase_gemm_mxint8_tn_packed (weight as int8 codes + scale bytes, widened in registers) against
    mase_gemm_bf16_tn(_packed) on the dequantized weight: the operands the matrix instruction sees are the same bf16
    values and the products are added in the same order, so the results are bit-identical, for every output dtype, with
    a bias, ragged M and N, several launches"""
    from mase_amd._gemm import gemm_bf16_pack_b, gemm_bf16_tn, gemm_mxint8_pack_b, gemm_mxint8_tn_packed
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(M + N + K + 1)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    w = torch.randn(N, K, generator=g) * 0.05
    w[::7] *= torch.exp2(torch.randint(-6, 7, (K,), generator=g).float())   # a wide range of block scales
    w[3] = 0.0
    bias = torch.randn(N, generator=g).to(dev)
    print(f"mxint8-codes gemm M={M} N={N} K={K}", flush=True)
    deq, codes, scales = _ops.mxint_qdq(w.to(dev), 32, 8, 1, 8, pack=True, out_dtype=torch.bfloat16)
    img, simg = gemm_mxint8_pack_b(codes.view(N, K), scales.view(N, K // 32))
    assert img.numel() == (N + 31) // 32 * 32 * K and simg.numel() == (N + 63) // 64 * 64 * (K // 32)
    from mase_amd import _lib

    # a few hundred rows: gemm_bf16_tn cuts K into ranges there and adds the partial sums in another order
    split = _lib.load().mase_gemm_bf16_tn_splitk_workspace_bytes(M, N, K) > 0
    bp = gemm_bf16_pack_b(deq.view(N, K))
    for dt, bs in ((torch.float32, None), (torch.bfloat16, bias), (torch.float16, bias.to(torch.float16))):
        want = gemm_bf16_tn(a, deq.view(N, K), bs, dt, b_packed=bp)
        for rep in range(3 if M * N * K > (1 << 36) else 2):
            got = gemm_mxint8_tn_packed(a, img, simg, N, bs, dt)
            if split:
                tol = 1e-5 if dt == torch.float32 else 1e-2
                assert float((got.float() - want.float()).abs().max() / want.float().abs().max()) < tol, (dt, rep)
            else:
                assert torch.equal(got, want), (dt, rep, float((got.float() - want.float()).abs().max()))


@pytest.mark.parametrize("B,H,S,T,D", [(2, 3, 100, 72, 64), (1, 4, 256, 256, 128), (2, 8, 520, 300, 128), (1, 1, 1, 64, 64),
                                       (3, 5, 33, 513, 192)])
def test_gemm_bf16_tn_batched_on_attention_layouts(dev, B, H, S, T, D):
    """The two contractions of an attention block on the layouts the modules hand over: query and output as [batch,
    heads, tokens, d] views of [batch, tokens, heads, d] memory, keys contiguous per head.  Small-integer operands make
    every partial sum exact, so each product must equal the integer product bit for bit; random operands are held
    to the rounding of the bf16 output against a float64 product."""
    from mase_amd._gemm import gemm_bf16_tn_batched, gemm_bf16_tn_batched_supported, matmul_bf16

    g = torch.Generator().manual_seed(B * 100 + S + T)
    print(f"batched gemm B={B} H={H} S={S} T={T} D={D}", flush=True)
    qi = torch.randint(-8, 9, (B, S, H, D), generator=g).float()
    ki = torch.randint(-8, 9, (B, H, T, D), generator=g).float()
    q = qi.bfloat16().to(dev).transpose(1, 2)          # [B, H, S, D] view, row stride H * D
    k = ki.bfloat16().to(dev)
    assert gemm_bf16_tn_batched_supported(q, k)
    want = qi.transpose(1, 2) @ ki.transpose(-1, -2)   # exact: |sums| <= 64 * D
    for dt in (torch.float32, torch.bfloat16):
        got = gemm_bf16_tn_batched(q, k, out_dtype=dt)
        assert got.shape == (B, H, S, T) and got.dtype == dt
        assert torch.equal(got.cpu().float(), want.to(dt).float())
    # scores x values through matmul_bf16 (values [B, H, T, D] are copied into rows of T; T is padded to a multiple of
    # 64 when it is not one), written into [B, S, H, D] memory
    pi = torch.randint(0, 5, (B, H, S, T), generator=g).float()
    vi = torch.randint(-8, 9, (B, T, H, D), generator=g).float()
    p, v = pi.bfloat16().to(dev), vi.bfloat16().to(dev).transpose(1, 2)
    out = torch.full((B, S, H, D), 7.0, dtype=torch.bfloat16, device=dev)
    r = matmul_bf16(p, v, out=out.transpose(1, 2))
    assert r is not None and r.data_ptr() == out.data_ptr()
    assert torch.equal(out.cpu().float(), (pi @ vi.transpose(1, 2)).transpose(1, 2).bfloat16().float())
    # random operands
    a = torch.randn(B, H, S, D, generator=g).bfloat16()
    b = torch.randn(B, H, T, D, generator=g).bfloat16()
    ref = a.double() @ b.double().transpose(-1, -2)
    assert rel_err(gemm_bf16_tn_batched(a.to(dev), b.to(dev), out_dtype=torch.float32).cpu(), ref) < 2e-6
    assert rel_err(gemm_bf16_tn_batched(a.to(dev), b.to(dev)).cpu(), ref) < 4e-3


def test_matmul_bf16_shapes_it_takes_and_leaves(dev):
    from mase_amd._gemm import matmul_bf16

    g = torch.Generator().manual_seed(3)
    x = torch.randint(-4, 5, (6, 40, 100), generator=g).float()     # contraction length 100: padded to 128
    y = torch.randint(-4, 5, (6, 100, 24), generator=g).float()
    got = matmul_bf16(x.bfloat16().to(dev), y.bfloat16().to(dev), out_dtype=torch.float32)
    assert got.shape == (6, 40, 24) and torch.equal(got.cpu(), x @ y)
    got16 = matmul_bf16(x.bfloat16().to(dev), y.bfloat16().to(dev))   # 24 bf16 = 48 bytes per row: a whole number of pieces
    assert torch.equal(got16.cpu().float(), (x @ y).bfloat16().float())
    y1 = torch.randint(-4, 5, (6, 100, 3), generator=g).float()      # 3 bf16 per row: the result's rows are padded
    got3 = matmul_bf16(x.bfloat16().to(dev), y1.bfloat16().to(dev))
    assert got3.shape == (6, 40, 3) and torch.equal(got3.cpu().float(), (x @ y1).bfloat16().float())
    # not taken: broadcast leading dimensions, other dtypes, 2-D operands, CPU tensors
    assert matmul_bf16(x[:1].bfloat16().to(dev), y.bfloat16().to(dev)) is None
    assert matmul_bf16(x.to(dev), y.to(dev)) is None
    assert matmul_bf16(x[0].bfloat16().to(dev), y[0].bfloat16().to(dev)) is None
    assert matmul_bf16(x.bfloat16(), y.bfloat16()) is None


def test_batched_gemm_c_abi_checks(dev):
    from mase_amd import _lib

    lib = _lib.load()
    a = torch.zeros(2, 64, 64, device=dev).bfloat16()
    c = torch.zeros(2, 64, 64, device=dev).bfloat16()
    call = lambda **kw: lib.mase_gemm_bf16_tn_batched(*[{**dict(A=a.data_ptr(), B=a.data_ptr(), C=c.data_ptr(), bo=1, bi=2, M=64, N=64,
                                                                K=64, lda=64, ldb=64, ldc=64, aso=0, asi=4096, bso=0, bsi=4096,
                                                                cso=0, csi=4096, dt=1, st=None), **kw}[k]
                                                         for k in ("A", "B", "C", "bo", "bi", "M", "N", "K", "lda", "ldb", "ldc", "aso",
                                                                   "asi", "bso", "bsi", "cso", "csi", "dt", "st")])
    assert call() == 0
    assert call(K=96) == -2 and call(lda=32) == -2 and call(ldc=60) == -2       # shape
    assert call(lda=68) == -3 and call(csi=4100) == -3 and call(A=a.data_ptr() + 2) == -3   # alignment
    assert call(A=None) == -1 and call(dt=5) == -4
    assert call(bo=0) == 0 and call(M=0) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_transpose_last2_with_zero_padding(dev, dtype):
    """mase_transpose16 against the tensor operation: views of [batch, tokens, heads, d] memory, ragged row counts
    (padded with zeros to a multiple of 64), column counts that are not a multiple of the 64-wide tile, 3-D operands"""
    from mase_amd import _gemm

    g = torch.Generator().manual_seed(21)
    cases = [torch.randn(2, 70, 3, 128, generator=g).to(dtype).to(dev).transpose(1, 2),   # [2, 3, 70, 128] view
             torch.randn(5, 200, 72, generator=g).to(dtype).to(dev),
             torch.randn(1, 2, 64, 8, generator=g).to(dtype).to(dev),
             torch.randn(4, 130, 136, generator=g).to(dtype).to(dev)[:, :, :104]]
    for y in cases:
        K = y.shape[-2]
        padded = (K + 63) // 64 * 64
        got = _gemm.transpose_last2(y, padded)
        assert got.shape == y.shape[:-2] + (y.shape[-1], padded) and got.is_contiguous()
        assert torch.equal(got[..., :K], y.transpose(-1, -2))
        assert bool((got[..., K:] == 0).all())
    # what the kernel does not take goes through the library's copy with the same result
    odd = torch.randn(3, 50, 12, generator=g).to(dtype).to(dev)      # 12 columns: not a multiple of 8
    got = _gemm.transpose_last2(odd, 64)
    assert torch.equal(got[..., :50], odd.transpose(-1, -2)) and bool((got[..., 50:] == 0).all())
    lib = _gemm._lib.load()
    a = torch.zeros(64, 64, dtype=dtype, device=dev)
    assert lib.mase_transpose16(a.data_ptr(), a.data_ptr(), 1, 1, 64, 12, 64, 0, 0, 64, None) == -2
    assert lib.mase_transpose16(a.data_ptr(), a.data_ptr(), 1, 1, 60, 64, 128, 0, 0, 64, None) == -2
    assert lib.mase_transpose16(a.data_ptr(), a.data_ptr(), 1, 1, 64, 64, 64, 0, 0, 60, None) == -2
    assert lib.mase_transpose16(a.data_ptr(), a.data_ptr(), 1, 1, 64, 64, 64, 4, 0, 64, None) == -3
    assert lib.mase_transpose16(None, a.data_ptr(), 1, 1, 64, 64, 64, 0, 0, 64, None) == -1
