"""Functional quantized Linear forms for the formats whose weights are quantized on every call.

Same names, config keys and behaviour as the reference's ``chop/nn/quantized/functional/linear.py``
(``linearInteger`` :24-73, ``linearMinifloatDenorm`` :76-123, ``linearMinifloatIEEE`` :126-173,
``linearBlockFP`` :220-278): quantize x, W and b, then one dense ``F.linear``.  The quantizers are the HIP
kernels; the contraction of already-dequantized operands is a plain library GEMM (rocBLAS/hipBLASLt through
``F.linear``) in the tensors' own dtype, exactly the operation the reference performs at that point.
"""
from __future__ import annotations

from functools import partial

from torch import Tensor
from torch.nn import functional as F

from ...quantizers import (
    block_fp_quantizer,
    integer_floor_quantizer,
    integer_quantizer,
    minifloat_denorm_quantizer,
    minifloat_ieee_quantizer,
)


def linearInteger(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None, out_config: dict = None):
    w_width, w_frac_width = config["weight_width"], config["weight_frac_width"]
    x_width, x_frac_width = config["data_in_width"], config["data_in_frac_width"]
    b_width, b_frac_width = config["bias_width"], config["bias_frac_width"]
    if out_config is not None:
        out_width, out_frac_width = out_config["data_out_width"], out_config["data_out_frac_width"]
    elif "data_out_width" in config:
        out_width, out_frac_width = config["data_out_width"], config["data_out_frac_width"]

    floor = config.get("floor", False)
    base_quantizer = integer_floor_quantizer if floor else integer_quantizer
    x = base_quantizer(x, width=x_width, frac_width=x_frac_width)
    weight = base_quantizer(weight, width=w_width, frac_width=w_frac_width)
    bias = base_quantizer(bias, width=b_width, frac_width=b_frac_width) if bias is not None else None
    out = F.linear(x, weight, bias)
    if "data_out_width" in config or out_config is not None:
        out = base_quantizer(out, width=out_width, frac_width=out_frac_width)
    return out


def _linear_minifloat(quantizer, x, weight, bias, config):
    wq = partial(quantizer, width=config["weight_width"], exponent_width=config["weight_exponent_width"],
                 exponent_bias=config["weight_exponent_bias"])
    xq = partial(quantizer, width=config["data_in_width"], exponent_width=config["data_in_exponent_width"],
                 exponent_bias=config["data_in_exponent_bias"])
    bq = partial(quantizer, width=config["bias_width"], exponent_width=config["bias_exponent_width"],
                 exponent_bias=config["bias_exponent_bias"])
    x = xq(x)
    weight = wq(weight)
    bias = bq(bias) if bias is not None else None
    return F.linear(x, weight, bias)


def linearMinifloatDenorm(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None):
    return _linear_minifloat(minifloat_denorm_quantizer, x, weight, bias, config)


def linearMinifloatIEEE(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None):
    return _linear_minifloat(minifloat_ieee_quantizer, x, weight, bias, config)


def linearBlockFP(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None):
    w_cfg = (config["weight_width"], config["weight_exponent_width"], config["weight_exponent_bias"],
             config["weight_block_size"])
    x_cfg = (config["data_in_width"], config["data_in_exponent_width"], config["data_in_exponent_bias"],
             config["data_in_block_size"])
    x_skip_first_dim = config.get("data_in_skip_first_dim", True)
    b_cfg = (config["bias_width"], config["bias_exponent_width"], config["bias_exponent_bias"],
             config["bias_block_size"])
    x = block_fp_quantizer(x, *x_cfg, skip_first_dim=x_skip_first_dim)
    weight = block_fp_quantizer(weight, *w_cfg, skip_first_dim=False)
    bias = block_fp_quantizer(bias, *b_cfg, skip_first_dim=False) if bias is not None else None
    return F.linear(x, weight, bias)
