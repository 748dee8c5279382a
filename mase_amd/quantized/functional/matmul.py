"""``matmul_mxint`` / ``matmul_mxfp`` / ``bmm_mxint`` / ``bmm_mxfp`` with the names, config keys and behaviour of the
reference's ``chop/nn/quantized/functional/matmul.py:437-512``: both operands are MX-quantized along their *last*
dimension (``block_dim=-1``; for ``y`` that is N, not the contraction dimension), then multiplied.

The quantizers are the HIP kernels.  A product whose quantized operands are exact in bf16 (MXINT up to 8 bits, every
MXFP format) runs on the bf16 matrix-core kernel of this package with fp32 accumulation: 2-D operands on
``mase_gemm_bf16_tn``, batched operands with equal leading dimensions on ``mase_gemm_bf16_tn_batched``.  Anything else
(broadcast leading dimensions, wider mantissas, gradients recorded) goes to ``torch.matmul`` / ``torch.bmm`` as in the
reference.
"""
from __future__ import annotations

from functools import partial

import torch

from ..._gemm import gemm_bf16_tn, matmul_bf16
from ...quantizers import mxfp_quantizer, mxint_quantizer

matmul_mapping = {"matmul": torch.matmul, "bmm": torch.bmm}


def _product(x, y, style, exact_in_bf16):
    if (style == "matmul" and exact_in_bf16 and x.dim() == 2 and y.dim() == 2 and x.is_cuda and x.dtype == y.dtype
            and x.dtype in (torch.float32, torch.bfloat16, torch.float16) and x.numel() > 0 and y.numel() > 0
            and not (torch.is_grad_enabled() and (x.requires_grad or y.requires_grad))):
        return gemm_bf16_tn(x.to(torch.bfloat16), y.t().to(torch.bfloat16), None, x.dtype)
    if (exact_in_bf16 and x.dim() == y.dim() >= 3 and x.is_cuda and x.dtype == y.dtype
            and x.dtype in (torch.float32, torch.bfloat16, torch.float16)
            and not (torch.is_grad_enabled() and (x.requires_grad or y.requires_grad))):
        out = matmul_bf16(x.to(torch.bfloat16), y.to(torch.bfloat16), out_dtype=x.dtype)
        if out is not None:
            return out
    return matmul_mapping[style](x, y)


def generic_matmul_mxfp(x, y, config, style="matmul"):
    if config.get("bypass", False):
        return matmul_mapping[style](x, y)
    x_quantizer = partial(mxfp_quantizer, block_size=config["data_in_block_size"],
                          element_exp_bits=config["data_in_exponent_width"],
                          element_frac_bits=config["data_in_frac_width"], block_dim=-1)
    y_quantizer = partial(mxfp_quantizer, block_size=config["weight_block_size"],
                          element_exp_bits=config["weight_exponent_width"],
                          element_frac_bits=config["weight_frac_width"], block_dim=-1)
    return _product(x_quantizer(x), y_quantizer(y), style, True)


def generic_matmul_mxint(x, y, config, style="matmul"):
    if config.get("bypass", False):
        return matmul_mapping[style](x, y)
    x_quantizer = partial(mxint_quantizer, block_size=config["data_in_block_size"],
                          element_bits=config["data_in_width"], block_dim=-1)
    y_quantizer = partial(mxint_quantizer, block_size=config["weight_block_size"],
                          element_bits=config["weight_width"], block_dim=-1)
    exact = max(config["data_in_width"], config["weight_width"]) <= 8
    return _product(x_quantizer(x), y_quantizer(y), style, exact)


def matmul_mxfp(x, y, config):
    return generic_matmul_mxfp(x, y, config, "matmul")


def matmul_mxint(x, y, config):
    return generic_matmul_mxint(x, y, config, "matmul")


def bmm_mxfp(x, y, config):
    return generic_matmul_mxfp(x, y, config, "bmm")


def bmm_mxint(x, y, config):
    return generic_matmul_mxint(x, y, config, "bmm")


quantized_func_map = {
    "matmul_mxfp": matmul_mxfp,
    "matmul_mxint": matmul_mxint,
    "bmm_mxfp": bmm_mxfp,
    "bmm_mxint": bmm_mxint,
}
