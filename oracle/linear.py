"""CPU restatement of the quantized Linear forwards.  TEST INFRASTRUCTURE.

Citations: ``src/chop/nn/quantized/modules/linear.py`` (modules) and
``src/chop/nn/quantized/functional/linear.py`` (functional forms).
"""
from __future__ import annotations

from torch import Tensor
from torch.nn import functional as F

from . import quantizers as Q


def mxint_prepare_weights(weight: Tensor, bias: Tensor | None, config: dict):
    """What ``LinearMXInt.load_state_dict`` leaves in ``.weight``/``.bias`` (modules/linear.py:916-954)."""
    if config.get("bypass", False) or config.get("gptq", False):
        return weight, bias
    w = Q.mxint_quantizer(weight, block_size=config["weight_block_size"], element_bits=config["weight_width"], block_dim=1)
    bb, bw = config.get("bias_block_size"), config.get("bias_width")
    if bias is not None and bb is not None and bw is not None:
        bias = Q.mxint_quantizer(bias, block_size=bb, element_bits=bw, block_dim=0)
    return w, bias


def linear_mxint_forward(x: Tensor, qweight: Tensor, qbias: Tensor | None, config: dict) -> Tensor:
    """``LinearMXInt.forward`` (modules/linear.py:956-972) on already-prepared weights."""
    if config.get("bypass", False):
        return F.linear(x, qweight, qbias)
    bs, bits = config.get("data_in_block_size"), config.get("data_in_width")
    if bs is not None and bits is not None:
        x = Q.mxint_quantizer(x, block_size=bs, element_bits=bits, block_dim=-1)
    return F.linear(x, qweight, qbias)


def mxfp_prepare_weights(weight: Tensor, bias: Tensor | None, config: dict):
    """``LinearMXFP.load_state_dict`` (modules/linear.py:835-875)."""
    if config.get("bypass", False) or config.get("gptq", False):
        return weight, bias
    w = Q.mxfp_quantizer(
        weight,
        block_size=config["weight_block_size"],
        element_exp_bits=config["weight_exponent_width"],
        element_frac_bits=config["weight_frac_width"],
        block_dim=1,
    )
    bb, be, bf = config.get("bias_block_size"), config.get("bias_exponent_width"), config.get("bias_frac_width")
    if bias is not None and bb is not None and be is not None:
        bias = Q.mxfp_quantizer(bias, block_size=bb, element_exp_bits=be, element_frac_bits=bf, block_dim=0)
    return w, bias


def linear_mxfp_forward(x: Tensor, qweight: Tensor, qbias: Tensor | None, config: dict) -> Tensor:
    """``LinearMXFP.forward`` (modules/linear.py:877-895)."""
    if config.get("bypass", False):
        return F.linear(x, qweight, qbias)
    bs, eb, fb = config.get("data_in_block_size"), config.get("data_in_exponent_width"), config.get("data_in_frac_width")
    if bs is not None and eb is not None:
        x = Q.mxfp_quantizer(x, block_size=bs, element_exp_bits=eb, element_frac_bits=fb, block_dim=-1)
    return F.linear(x, qweight, qbias)


def linear_integer(x: Tensor, weight: Tensor, bias: Tensor | None, config: dict, out_config: dict | None = None) -> Tensor:
    """``linearInteger`` (functional/linear.py:24-73)."""
    base = Q.integer_floor_quantizer if config.get("floor", False) else Q.integer_quantizer
    xq = base(x, config["data_in_width"], config["data_in_frac_width"])
    wq = base(weight, config["weight_width"], config["weight_frac_width"])
    bw, bf = config["bias_width"], config["bias_frac_width"]
    bq = base(bias, bw, bf) if bias is not None else None
    out = F.linear(xq, wq, bq)
    if "data_out_width" in config:
        out = base(out, config["data_out_width"], config["data_out_frac_width"])
    elif out_config is not None:
        out = base(out, out_config["data_out_width"], out_config["data_out_frac_width"])
    return out


def _linear_minifloat(fn, x, weight, bias, config):
    xq = fn(x, config["data_in_width"], config["data_in_exponent_width"], config["data_in_exponent_bias"])
    wq = fn(weight, config["weight_width"], config["weight_exponent_width"], config["weight_exponent_bias"])
    bcfg = (config["bias_width"], config["bias_exponent_width"], config["bias_exponent_bias"])
    bq = fn(bias, *bcfg) if bias is not None else None
    return F.linear(xq, wq, bq)


def linear_minifloat_denorm(x, weight, bias, config):
    """``linearMinifloatDenorm`` (functional/linear.py:76-123)."""
    return _linear_minifloat(Q.minifloat_denorm_quantizer, x, weight, bias, config)


def linear_minifloat_ieee(x, weight, bias, config):
    """``linearMinifloatIEEE`` (functional/linear.py:126-173)."""
    return _linear_minifloat(Q.minifloat_ieee_quantizer, x, weight, bias, config)


def linear_block_fp(x: Tensor, weight: Tensor, bias: Tensor | None, config: dict) -> Tensor:
    """``linearBlockFP`` (functional/linear.py:220-278)."""
    xq = Q.block_fp_quantizer(
        x, config["data_in_width"], config["data_in_exponent_width"], config["data_in_exponent_bias"],
        config["data_in_block_size"], skip_first_dim=config.get("data_in_skip_first_dim", True),
    )
    wq = Q.block_fp_quantizer(
        weight, config["weight_width"], config["weight_exponent_width"], config["weight_exponent_bias"],
        config["weight_block_size"], skip_first_dim=False,
    )
    bcfg = (config["bias_width"], config["bias_exponent_width"], config["bias_exponent_bias"], config["bias_block_size"])
    bq = Q.block_fp_quantizer(bias, *bcfg, skip_first_dim=False) if bias is not None else None
    return F.linear(xq, wq, bq)
