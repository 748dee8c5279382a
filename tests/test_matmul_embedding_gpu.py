"""GPU parity of the callers next to the Linear path: MX matmul / bmm functions and MX embeddings."""
import pytest
import torch

from oracle import matmul as OM
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu

MXINT = {"data_in_block_size": 32, "data_in_width": 8, "weight_block_size": 32, "weight_width": 8}
MXFP = {"data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3,
        "weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1}


def rel_err(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matmul_and_bmm_mx(dev, dtype):
    from mase_amd.quantized import bmm_mxfp, bmm_mxint, matmul_mxfp, matmul_mxint, quantized_func_map

    assert set(quantized_func_map) == {"matmul_mxint", "matmul_mxfp", "bmm_mxint", "bmm_mxfp"}
    g = torch.Generator().manual_seed(11)
    x2 = torch.randn(96, 128, generator=g).to(dtype)
    y2 = torch.randn(128, 160, generator=g).to(dtype)          # quantized along its last dim (160 = 5 blocks)
    x3 = torch.randn(6, 40, 64, generator=g).to(dtype)
    y3 = torch.randn(6, 64, 96, generator=g).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    with torch.no_grad():
        assert rel_err(matmul_mxint(x2.to(dev), y2.to(dev), MXINT), OM.matmul_mxint(x2, y2, MXINT)) < tol
        assert rel_err(matmul_mxfp(x2.to(dev), y2.to(dev), MXFP), OM.matmul_mxfp(x2, y2, MXFP)) < tol
        assert rel_err(matmul_mxint(x3.to(dev), y3.to(dev), MXINT), OM.matmul_mxint(x3, y3, MXINT)) < tol
        assert rel_err(bmm_mxint(x3.to(dev), y3.to(dev), MXINT), OM.matmul_mxint(x3, y3, MXINT, "bmm")) < tol
        assert rel_err(bmm_mxfp(x3.to(dev), y3.to(dev), MXFP), OM.matmul_mxfp(x3, y3, MXFP, "bmm")) < tol
        # bypass = plain product
        assert rel_err(matmul_mxint(x2.to(dev), y2.to(dev), {"bypass": True}), x2.float() @ y2.float()) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_mx_quantizes_only_looked_up_rows_bit_exactly(dev, dtype):
    from mase_amd.quantized import EmbeddingMXFP, EmbeddingMXInt, quantized_module_map

    assert quantized_module_map["embedding_mxint"] is EmbeddingMXInt and quantized_module_map["embedding_mxfp"] is EmbeddingMXFP
    g = torch.Generator().manual_seed(12)
    table = (torch.randn(500, 128, generator=g) * 0.05).to(dtype)
    idx = torch.randint(0, 500, (4, 37), generator=g)
    idx[0, :3] = 7
    for cls, cfg, ref_fn in ((EmbeddingMXInt, {"weight_block_size": 32, "weight_width": 8}, OM.embedding_mxint),
                             (EmbeddingMXFP, {"weight_block_size": 32, "weight_exponent_width": 4, "weight_frac_width": 3},
                              OM.embedding_mxfp)):
        m = cls(500, 128, config=dict(cfg), padding_idx=7, device=dev, dtype=dtype)
        with torch.no_grad():
            m.weight.copy_(table.to(dev))
        got = m(idx.to(dev))
        assert_bits_equal(got, ref_fn(idx, table, cfg, padding_idx=7), cls.__name__)
        assert got.shape == (4, 37, 128)
        assert m(torch.zeros(0, dtype=torch.long, device=dev)).shape == (0, 128)
        # a row length that is not a whole number of blocks keeps the reference's whole-table order
        m2 = cls(40, 48, config={**cfg, "weight_block_size": 16}, device=dev, dtype=dtype)
        with torch.no_grad():
            m2.weight.copy_(table[:40, :48].to(dev))
        assert_bits_equal(m2(idx.to(dev) % 40), ref_fn(idx % 40, table[:40, :48].contiguous(), {**cfg, "weight_block_size": 16}),
                          cls.__name__ + " small")
        # bypass
        mb = cls(500, 128, config={"bypass": True}, device=dev, dtype=dtype)
        with torch.no_grad():
            mb.weight.copy_(table.to(dev))
        assert_bits_equal(mb(idx.to(dev)), table[idx], "bypass")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantized_softmax_silu_rope_kvcache(dev, dtype):
    """thin callers of the quantizers (reference functional/softmax.py, silu.py, rope.py, kvcache.py): the quantized
    tensors are compared bit-exactly, the torch op applied on top within the library's CPU/GPU difference"""
    import oracle as O
    from mase_amd.quantized import functional as QF

    g = torch.Generator().manual_seed(13)
    x = (torch.randn(2, 4, 48, 64, generator=g) * 3).to(dtype)
    fcfg = {"data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}
    icfg = {"data_in_block_size": 32, "data_in_width": 8}
    mcfg = {"data_in_exponent_width": 4, "data_in_frac_width": 3}
    q_fp = lambda t: O.mxfp_quantizer(t, 32, 4, 3)
    q_int = lambda t: O.mxint_quantizer(t, 32, 8)
    q_mf = lambda t: O.minifloat_quantizer_sim(t, 4, 3, True, "rn", None)
    sm = lambda t: torch.softmax(t.float(), -1).to(t.dtype)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    xd = x.to(dev)
    for fn, q, cfg in ((QF.softmax_mxfp, q_fp, fcfg), (QF.softmax_mxint, q_int, icfg), (QF.softmax_minifloat, q_mf, mcfg)):
        assert rel_err(fn(xd, cfg), sm(q(x))) < tol
    for fn, q, cfg in ((QF.silu_mxfp, q_fp, fcfg), (QF.silu_mxint, q_int, icfg), (QF.silu_minifloat, q_mf, mcfg)):
        assert rel_err(fn(xd, cfg), torch.nn.functional.silu(q(x))) < tol
    k, v = QF.kv_cache_mxfp(xd, xd * 0.5, fcfg)
    assert_bits_equal(k, q_fp(x), "kv_cache_mxfp k")
    assert_bits_equal(v, q_fp(x * 0.5), "kv_cache_mxfp v")
    k, v = QF.kv_cache_mxint(xd, xd * 0.5, icfg)
    assert_bits_equal(k, q_int(x), "kv_cache_mxint k")
    # rotary embedding: cos/sin tables quantized, q/k untouched
    t = torch.arange(48, dtype=torch.float32)
    freqs = torch.outer(t, 1.0 / (10000 ** (torch.arange(0, 64, 2).float() / 64)))
    emb = torch.cat((freqs, freqs), -1)
    cos, sin = emb.cos()[None].to(dtype), emb.sin()[None].to(dtype)
    for fn, q, cfg in ((QF.rope_mxfp, q_fp, fcfg), (QF.rope_mxint, q_int, icfg), (QF.rope_minifloat, q_mf, mcfg)):
        qe, ke = fn(xd, xd * 2, cos.to(dev), sin.to(dev), cfg)
        c, s_ = q(cos).unsqueeze(1), q(sin).unsqueeze(1)
        rot = lambda u: torch.cat((-u[..., 32:], u[..., :32]), -1)
        assert rel_err(qe, x * c + rot(x) * s_) < tol and rel_err(ke, (x * 2) * c + rot(x * 2) * s_) < tol


def test_batched_products_run_on_the_kernel_of_this_package(dev, monkeypatch):
    """bmm_mx* and matmul_mx* on batched operands: the quantized operands are exact in bf16, so the product runs on
    mase_gemm_bf16_tn_batched whatever the tensors' dtype (fp32 results keep fp32 accumulation, rounded once);
    9-bit MXINT mantissas and broadcast leading dimensions stay with torch."""
    from mase_amd import _gemm
    from mase_amd.quantized import bmm_mxint, matmul_mxfp, matmul_mxint

    calls = []
    real = _gemm.gemm_bf16_tn_batched
    monkeypatch.setattr(_gemm, "gemm_bf16_tn_batched", lambda a, b, **kw: (calls.append(kw.get("out_dtype")), real(a, b, **kw))[1])
    g = torch.Generator().manual_seed(13)
    x = torch.randn(4, 50, 96, generator=g)
    y = torch.randn(4, 96, 64, generator=g)
    with torch.no_grad():
        for dtype in (torch.float32, torch.bfloat16):
            xd, yd = x.to(dtype).to(dev), y.to(dtype).to(dev)
            calls.clear()
            got = bmm_mxint(xd, yd, MXINT)
            assert calls == [dtype] and got.dtype == dtype
            assert rel_err(got, OM.matmul_mxint(x.to(dtype), y.to(dtype), MXINT, "bmm")) < (1e-5 if dtype == torch.float32 else 1e-2)
            matmul_mxfp(xd, yd, MXFP)
            assert len(calls) == 2
        calls.clear()
        wide = dict(MXINT, data_in_width=9)
        matmul_mxint(x.to(dev), y.to(dev), wide)            # 9-bit mantissas are not bf16 values
        matmul_mxint(x[:1].to(dev), y.to(dev), MXINT)        # broadcast over the batch
        assert calls == []
