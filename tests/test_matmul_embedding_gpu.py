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
