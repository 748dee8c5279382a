"""CPU restatement of the MX matmul / bmm functions and MX embeddings.  TEST INFRASTRUCTURE ONLY.

``matmul_mxint/mxfp``, ``bmm_mxint/mxfp``: reference ``chop/nn/quantized/functional/matmul.py:437-512`` — both
operands quantized along their last dimension, then ``torch.matmul`` / ``torch.bmm``.
``embedding_mxint/mxfp``: reference ``chop/nn/quantized/modules/embedding.py:9-71`` — the whole table quantized along
dim 1, then ``F.embedding``.  Pinned by composition: the quantizers are pinned in ``oracle.quantizers``; the
product and the lookup are library routines.
"""
import torch
from torch.nn import functional as F

from .quantizers import mxfp_quantizer, mxint_quantizer


def matmul_mxint(x, y, config, style="matmul"):
    xq = mxint_quantizer(x, config["data_in_block_size"], config["data_in_width"], block_dim=-1)
    yq = mxint_quantizer(y, config["weight_block_size"], config["weight_width"], block_dim=-1)
    return (torch.bmm if style == "bmm" else torch.matmul)(xq, yq)


def matmul_mxfp(x, y, config, style="matmul"):
    xq = mxfp_quantizer(x, config["data_in_block_size"], config["data_in_exponent_width"], config["data_in_frac_width"],
                        block_dim=-1)
    yq = mxfp_quantizer(y, config["weight_block_size"], config["weight_exponent_width"], config["weight_frac_width"],
                        block_dim=-1)
    return (torch.bmm if style == "bmm" else torch.matmul)(xq, yq)


def embedding_mxint(idx, weight, config, padding_idx=None):
    return F.embedding(idx, mxint_quantizer(weight, config["weight_block_size"], config["weight_width"], block_dim=1),
                       padding_idx)


def embedding_mxfp(idx, weight, config, padding_idx=None):
    wq = mxfp_quantizer(weight, config["weight_block_size"], config["weight_exponent_width"], config["weight_frac_width"],
                        block_dim=1)
    return F.embedding(idx, wq, padding_idx)
