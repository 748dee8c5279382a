"""Functional quantized Linear forms for the formats whose weights are quantized on every call.

Same names, config keys and behaviour as the reference's ``chop/nn/quantized/functional/linear.py``
(``linearInteger`` :24-73, ``linearMinifloatDenorm`` :76-123, ``linearMinifloatIEEE`` :126-173,
``linearBlockFP`` :220-278): quantize x, W and b, then one dense ``F.linear``.  The quantizers are the HIP
kernels.  When the quantized operands are exactly representable in bf16 (at most 8 significant bits: integer and
block-FP widths up to 9, minifloat mantissas up to 7 or 8 bits) the contraction runs on the bf16 matrix-core kernel
with fp32 accumulation (inference only: under ``torch.no_grad()`` or with no tensor requiring grad), which computes
the same real-number dot products as ``F.linear`` on the dequantized operands; otherwise it is the library GEMM (``F.linear``) in the tensors' own dtype, the operation the reference
performs at that point.  One caveat of the bf16 form for fp32 tensors: block-FP and minifloat pass elements with
|x| <= 1e-8 through unquantized, and those are rounded to bf16 (absolute error below 4e-11 per element).
"""
from __future__ import annotations

from functools import partial

import torch
from torch import Tensor
from torch.nn import functional as F

from ..._gemm import gemm_bf16_tn

from ...quantizers import (
    block_fp_quantizer,
    integer_floor_quantizer,
    integer_quantizer,
    minifloat_denorm_quantizer,
    minifloat_ieee_quantizer,
)


def _contract(x: Tensor, weight: Tensor, bias: Tensor | None, exact_in_bf16: bool) -> Tensor:
    """``F.linear(x, weight, bias)`` for already quantized operands.  The matrix-core kernel has no backward: it is
    used only when no gradient is being recorded (inference); training keeps the differentiable library GEMM."""
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad
                                              or (bias is not None and bias.requires_grad))
    if needs_grad or not (exact_in_bf16 and x.is_cuda and weight.dim() == 2 and x.numel() > 0
                          and x.dtype == weight.dtype and x.dtype in (torch.float32, torch.bfloat16, torch.float16)):
        return F.linear(x, weight, bias)
    lead = x.shape[:-1]
    y = gemm_bf16_tn(x.reshape(-1, x.shape[-1]).to(torch.bfloat16), weight.to(torch.bfloat16), bias, x.dtype)
    return y.reshape(*lead, weight.shape[0])


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
    out = _contract(x, weight, bias, max(w_width, x_width) <= 9)
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
    # mantissa bits (plus the implicit one of the ieee flavour) of both operands
    sig = max(config["weight_width"] - config["weight_exponent_width"] - 1,
              config["data_in_width"] - config["data_in_exponent_width"] - 1) + (1 if quantizer is minifloat_ieee_quantizer else 0)
    return _contract(x, weight, bias, sig <= 8)


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
    return _contract(x, weight, bias, max(config["weight_width"], config["data_in_width"]) <= 9)
