"""One-pass RMSNorm and SiLU-product kernels against the separate tensor operations (torch on the GPU for the plain
forms, the CPU oracle for the minifloat-cast forms), and the sharing of quantized activations between projections."""
import pytest
import torch

import oracle as O
from oracle import llama as OL

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
ULP = {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def close_in_ulps(got, want, dtype, n_ulp, frac_equal):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs() / want.abs().clamp_min(1e-30)
    assert float(err.max()) <= n_ulp * ULP[dtype], float(err.max())
    assert float((got == want).float().mean()) >= frac_equal, float((got == want).float().mean())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols", [8, 256, 1536, 1600, 2048, 4096, 5120, 8192])
def test_rmsnorm_one_pass(dev, dtype, cols):
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(cols)
    x = (torch.randn(37, cols, generator=g) * 1.7).to(dtype)
    w = (1.0 + 0.2 * torch.randn(cols, generator=g)).to(dtype)
    xd, wd = x.to(dev), w.to(dev)
    assert _ops.rmsnorm_supported(xd, wd)
    got = _ops.rmsnorm_minifloat(xd, wd, 1e-6)
    h = xd.float()
    want = wd * (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)).to(dtype)
    # the row sum is taken in another order: a result may land on the neighbouring value of dtype
    close_in_ulps(got, want, dtype, 1.01 if dtype != torch.float32 else 8, 0.995 if dtype != torch.float32 else 0.5)
    # with casts: against the oracle's restatement of LlamaRMSNormMinifloat.forward
    qc = {"data_in_exponent_width": 4, "data_in_frac_width": 3, "weight_exponent_width": 5, "weight_frac_width": 2,
          "weight_round_mode": "ru"}
    got = _ops.rmsnorm_minifloat(xd, wd, 1e-6, (4, 3, True, "rn"), (5, 2, True, "ru"))
    close_in_ulps(got, OL.rms_norm_forward(w, x, 1e-6, qc), dtype, 1.01 if dtype != torch.float32 else 8,
                  0.995 if dtype != torch.float32 else 0.5)
    assert not _ops.rmsnorm_supported(xd, wd.float() if dtype != torch.float32 else wd.bfloat16())
    assert not _ops.rmsnorm_supported(xd[:, : cols - 4], wd[: cols - 4]) or (cols - 4) % 8 == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_one_pass(dev, dtype):
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(3)
    gate = (torch.randn(33, 1000, generator=g) * 3).to(dtype)
    up = torch.randn(33, 1000, generator=g).to(dtype)
    gate[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 88.0, -88.0, 1e-3, -1e-3]).to(dtype)
    got = _ops.silu_mul_minifloat(gate.to(dev), up.to(dev))
    want = torch.nn.functional.silu(gate.to(dev)) * up.to(dev)
    close_in_ulps(got, want, dtype, 2.02 if dtype != torch.float32 else 8, 0.99 if dtype != torch.float32 else 0.5)
    got = _ops.silu_mul_minifloat(gate.to(dev), up.to(dev), (4, 3, True, "rn"))
    want = torch.nn.functional.silu(O.minifloat_quantizer_sim(gate, 4, 3, True, "rn")) * up
    close_in_ulps(got, want, dtype, 2.02 if dtype != torch.float32 else 8, 0.99 if dtype != torch.float32 else 0.5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_one_pass_is_bit_identical_to_the_tensor_operations(dev, dtype):
    """products and sum are single roundings of exact fp32 values on both sides: identical bits"""
    from mase_amd.quantizers import _ops
    from mase_amd.quantized.functional.activations import rope_minifloat, rotate_half

    g = torch.Generator().manual_seed(9)
    B, T, H, D = 2, 50, 6, 64
    proj = torch.randn(B, T, H * D, generator=g).to(dtype).to(dev)
    q = proj.view(B, T, H, D).transpose(1, 2)                       # the strided view a projection output gives
    ang = torch.rand(B, T, D, generator=g) * 6.28
    cos, sin = ang.cos().to(dtype).to(dev), ang.sin().to(dtype).to(dev)
    for c, s_ in ((cos, sin), (cos[0], sin[0]), (cos[:1], sin[:1])):
        assert _ops.rope_supported(q, c, s_)
        got = _ops.rope(q, c, s_)
        cc, ss = (c, s_) if c.dim() == 2 else (c.unsqueeze(1), s_.unsqueeze(1))
        want = q * cc + rotate_half(q) * ss
        assert got.stride() == q.stride() and torch.equal(got, want)
    qc = q.contiguous()
    assert torch.equal(_ops.rope(qc, cos, sin), qc * cos.unsqueeze(1) + rotate_half(qc) * sin.unsqueeze(1))
    # the quantized caller: cos / sin through the minifloat cast, then the same kernel
    cfg = {"data_in_exponent_width": 4, "data_in_frac_width": 3}
    qq, kk = rope_minifloat(q, q * 0.5, cos, sin, cfg)
    cq = O.minifloat_quantizer_sim(cos.cpu(), 4, 3, True, "rn").to(dev).unsqueeze(1)
    sq = O.minifloat_quantizer_sim(sin.cpu(), 4, 3, True, "rn").to(dev).unsqueeze(1)
    assert torch.equal(qq, q * cq + rotate_half(q) * sq) and torch.equal(kk, (q * 0.5) * cq + rotate_half(q * 0.5) * sq)
    assert not _ops.rope_supported(q[..., :40], cos[..., :40], sin[..., :40])   # head_dim not a multiple of 16


def test_project_shared_quantizes_once_per_quantizer(dev, monkeypatch):
    """project_shared: one activation quantization for sibling projections with the same quantizer, one more for a
    module with another format; separate module calls quantize every time (nothing is remembered between calls)"""
    from mase_amd.quantized import LinearMXInt
    from mase_amd.quantized.functional.mx_linear import project_shared
    from mase_amd.quantizers import _ops

    cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}
    torch.manual_seed(0)
    mods = []
    for _ in range(3):
        m = LinearMXInt(256, 128, bias=False, device=dev, dtype=torch.bfloat16, config=dict(cfg))
        m.load_state_dict({"weight": torch.randn(128, 256) * 0.05})
        mods.append(m)
    other = LinearMXInt(256, 128, bias=False, device=dev, dtype=torch.bfloat16, config={**cfg, "data_in_width": 6})
    other.load_state_dict({"weight": torch.randn(128, 256) * 0.05})
    calls = []
    real = _ops.mxint_qdq
    monkeypatch.setattr(_ops, "mxint_qdq", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    x = torch.randn(300, 256, device=dev, dtype=torch.bfloat16)
    ys = project_shared(x, mods)
    assert len(calls) == 1                               # q/k/v style: one quantization for three projections
    ref = [m(x) for m in mods]                           # separate calls: quantized again each time
    assert len(calls) == 4
    for a, b in zip(ys, ref):
        assert torch.equal(a, b)
    n = len(calls)
    project_shared(x, mods + [other])                    # another activation format gets its own copy
    assert len(calls) == n + 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [8, 4])
def test_norm_and_silu_product_written_in_the_consumers_mxint_form(dev, dtype, bits):
    """mase_rmsnorm_mxint / mase_silu_mul_mxint: bit for bit the MXINT quantizer (checked against the oracle elsewhere)
    applied to what the unquantized kernels store; rows of awkward lengths, blocks of zeros, huge and tiny blocks"""
    from mase_amd.quantizers import _ops
    from helpers import assert_bits_equal

    g = torch.Generator().manual_seed(5 + bits)
    for rows, cols in ((37, 4096), (5, 32), (3, 5120), (130, 96), (2, 8192), (9, 1536), (7, 1600), (4, 2048)):
        x = (torch.randn(rows, cols, generator=g) * 1.7).to(dtype)
        x[0, :32] = 0
        x[1 % rows, 32:64] *= 1e-3
        w = (1.0 + 0.2 * torch.randn(cols, generator=g)).to(dtype)
        w[:32] = 0  # a block of zeros after the norm
        xd, wd = x.to(dev), w.to(dev)
        want = _ops.mxint_qdq(_ops.rmsnorm_minifloat(xd, wd, 1e-6), 32, bits, -1, 8)
        assert_bits_equal(_ops.rmsnorm_mxint(xd, wd, 1e-6, bits), want, f"rmsnorm_mxint {dtype} {rows}x{cols}")
        # the residual addition in the same pass: the sum as the tensor addition rounds it, and the norm of that sum
        rd = (torch.randn(rows, cols, generator=g) * 0.9).to(dtype).to(dev)
        ssum, hq = _ops.add_rmsnorm_mxint(xd, rd, wd, 1e-6, bits)
        assert_bits_equal(ssum, xd + rd, f"add_rmsnorm_mxint sum {dtype} {rows}x{cols}")
        assert_bits_equal(hq, _ops.rmsnorm_mxint(xd + rd, wd, 1e-6, bits), f"add_rmsnorm_mxint norm {dtype} {rows}x{cols}")
        gate = (torch.randn(rows, cols, generator=g) * 3).to(dtype)
        up = torch.randn(rows, cols, generator=g).to(dtype)
        gate[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 88.0, -88.0, 1e-3, -1e-3]).to(dtype)
        up[-1, -32:] *= 1e4 if dtype != torch.float16 else 50.0
        gd, ud = gate.to(dev), up.to(dev)
        want = _ops.mxint_qdq(_ops.silu_mul_minifloat(gd, ud), 32, bits, -1, 8)
        assert_bits_equal(_ops.silu_mul_mxint(gd, ud, bits, use_table=False), want, f"silu_mul_mxint {dtype} {rows}x{cols}")
        if dtype != torch.float32:  # the form that reads silu from a table: the same bits
            assert_bits_equal(_ops.silu_mul_mxint(gd, ud, bits, use_table=True), want, f"silu_mul_mxint table {dtype} {rows}x{cols}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_table_form_for_every_gate_pattern_and_at_size(dev, dtype):
    """mase_silu_mul_mxint_lut against mase_silu_mul_mxint bit for bit: every 16-bit pattern as the gate (NaNs and
    infinities included), non-finite and huge second factors, a tensor large enough that the dispatch picks the table
    form by itself (more work-groups' worth of vectors than CUs, a ragged last wavefront)"""
    from mase_amd.quantizers import _ops
    from helpers import assert_bits_equal

    g = torch.Generator().manual_seed(17)
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).reshape(2048, 32).to(dev)
    for scale in (1.0, 1e3 if dtype == torch.float16 else 1e30):
        up = (torch.randn(2048, 32, generator=g) * scale).to(dtype).to(dev)
        up[5, 3] = float("inf")
        up[6, 4] = float("nan")
        for bits in (8, 4, 2):
            assert_bits_equal(_ops.silu_mul_mxint(gate, up, bits, use_table=True),
                              _ops.silu_mul_mxint(gate, up, bits, use_table=False), f"table form, all gates, {dtype} bits {bits}")
    rows, cols = 4099, 2144   # 8.8 M elements: above the dispatch threshold, not a multiple of the grid's stride
    assert rows * cols >= _ops.SILU_TABLE_MIN_NUMEL
    gate = (torch.randn(rows, cols, generator=g) * 2.5).to(dtype).to(dev)
    up = torch.randn(rows, cols, generator=g).to(dtype).to(dev)
    assert_bits_equal(_ops.silu_mul_mxint(gate, up, 8), _ops.silu_mul_mxint(gate, up, 8, use_table=False), f"table form at size, {dtype}")


# the last two: enough (batch, head) pairs per XCD for the persistent form of the kernel (2 and 4 items per work-group)
@pytest.mark.parametrize("B,H,T", [(1, 1, 128), (2, 3, 256), (1, 2, 640), (1, 4, 2048), (2, 4, 384), (1, 16, 256), (8, 64, 256),
                                   (2, 64, 1024)])
@pytest.mark.parametrize("layout", ["bthd", "bhtd"])
def test_causal_attention_one_pass(dev, B, H, T, layout):
    """mase_attention_causal against the tensor operations in fp32 (masked scores, softmax, product with v) on the same
    bf16 operands: bound 1e-2 of the output range (the probabilities are rounded to bf16 before the second product and
    the output is bf16); the library's own kernel is held to the same bound for comparison.  Operands as strided views
    of [batch, tokens, heads, 128] memory (what the projections produce) and contiguous [batch, heads, tokens, 128]."""
    from helpers import assert_bits_equal
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(B * 1000 + T)
    mk = lambda scale: (torch.randn(B, T, H, 128, generator=g) * scale).bfloat16().to(dev)
    q, k, v = mk(1.5), mk(1.0), mk(2.0)
    if layout == "bthd":
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    else:
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    assert _ops.attention_causal_supported(q, k, v)
    # scaling 0.6 spreads the scores over some hundred powers of two: the reference point of the exponentials moves in
    # most key blocks, and rows are close to one-hot
    for scaling in (None, 0.05, 0.6):
        sc = 128 ** -0.5 if scaling is None else scaling
        s = (q.float() @ k.float().transpose(-1, -2)) * sc
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool, device=dev), 1), float("-inf"))
        ref = torch.softmax(s, -1) @ v.float()
        got = _ops.attention_causal(q, k, v, scaling)
        assert got.shape == (B, H, T, 128) and got.dtype == torch.bfloat16
        assert got.transpose(1, 2).reshape(B, T, H * 128).data_ptr() == got.data_ptr()  # [B, T, H*128] is a view
        e = float((got.float() - ref).abs().max() / ref.abs().max())
        lib = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=sc)
        e_lib = float((lib.float() - ref).abs().max() / ref.abs().max())
        print(f"causal attention {B}x{H}x{T} {layout} scale {sc:.3f}: err {e:.2e} (library kernel {e_lib:.2e})")
        assert e < 1e-2
        # the first query attends to the first key only: its output row is v[0]
        assert torch.equal(got[:, :, 0], v[:, :, 0])
        # the MXINT output form: the quantizer's result on the stored bf16 output (oracle on the CPU), bit for bit
        for bits in (8, 4):
            gq = _ops.attention_causal(q, k, v, scaling, mxint_bits=bits).transpose(1, 2).reshape(B, T, H * 128)
            want = O.mxint_quantizer(got.transpose(1, 2).reshape(B, T, H * 128).cpu(), 32, bits, block_dim=-1)
            assert_bits_equal(gq, want, f"attention output as MXINT{bits}")
    # q handed over before its rotary embedding: the kernel's rotation on load gives the values of rope() followed by
    # the plain call, with and without the MXINT output form; tables shared by the batch and per batch item
    ang = torch.rand(T, 64, generator=g) * 6.28
    emb = torch.cat((ang, ang), -1)
    cos, sin = emb.cos().bfloat16().to(dev), emb.sin().bfloat16().to(dev)
    # per batch item: different angles for every item, so that a wrong batch stride of the tables shows
    ang_b = ang[None] * (1.0 + 0.37 * torch.arange(B)[:, None, None])
    emb_b = torch.cat((ang_b, ang_b), -1)
    per_item = (emb_b.cos().bfloat16().to(dev), (emb_b.sin() * 0.5).bfloat16().to(dev))
    assert B == 1 or not torch.equal(per_item[0][0], per_item[0][1])
    for tables in ((cos, sin), per_item):
        assert _ops.rope_supported(q, *tables)
        want = _ops.attention_causal(_ops.rope(q, *tables), k, v)
        assert torch.equal(_ops.attention_causal(q, k, v, q_rope=tables), want)
        assert torch.equal(_ops.attention_causal(q, k, v, mxint_bits=8, q_rope=tables),
                           _ops.attention_causal(_ops.rope(q, *tables), k, v, mxint_bits=8))
    assert not _ops.attention_causal_supported(q[:, :, :100], k[:, :, :100], v[:, :, :100])
    assert not _ops.attention_causal_supported(q.float(), k.float(), v.float())
    assert not _ops.attention_causal_supported(q[..., :64], k[..., :64], v[..., :64])
