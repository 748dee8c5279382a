"""Functional quantized Linear forms for the formats whose weights are quantized on every call.

Same names, config keys and behaviour as the reference's ``chop/nn/quantized/functional/linear.py``
(``linearInteger`` :24-73, ``linearMinifloatDenorm`` :76-123, ``linearMinifloatIEEE`` :126-173,
``linearBlockFP`` :220-278): quantize x, W and b, then one dense ``F.linear``.  The quantizers are the HIP
kernels.  When the quantized operands are exactly representable in bf16 (at most 8 significant bits: integer and
block-FP widths up to 9, minifloat mantissas up to 7 or 8 bits) the contraction runs on the bf16 matrix-core kernel
with fp32 accumulation (inference only: under ``torch.no_grad()`` or with no tensor requiring grad), which computes
the same real-number dot products as ``F.linear`` on the dequantized operands; otherwise it is the library GEMM (``F.linear``) in the tensors' own dtype, the operation the reference
performs at that point.  ``param_cache`` (keyword-only, not in the reference's signatures; the modules pass theirs when their config holds
``cache_quantized_params=True``) keeps the quantized parameters between inference calls instead of recomputing
identical tensors; without it weight and bias are quantized on every call, as in the reference.  One caveat of the bf16 form for fp32 tensors: block-FP and minifloat pass elements with
|x| <= 1e-8 through unquantized, and those are rounded to bf16 (absolute error below 4e-11 per element).
"""
from __future__ import annotations

from functools import partial

import torch
from torch import Tensor
from torch.nn import functional as F

from ..._gemm import gemm_bf16_pack_b, gemm_bf16_packed_b_supported, gemm_bf16_takes_packed_b, gemm_bf16_tn
from .mx_linear import _tensor_key as _observable_key

from ...quantizers import (
    block_fp_quantizer,
    integer_floor_quantizer,
    integer_quantizer,
    minifloat_denorm_quantizer,
    minifloat_ieee_quantizer,
)


def _tensor_key(t: Tensor | None):
    return "absent" if t is None else _observable_key(t)


class QuantizedParamCache:
    """The quantized weight and bias of a module whose reference form quantizes them again on every call, and the
    bf16 / fragment-ordered copies of that weight for the matrix-core kernel.  Parameters do not change between
    inference forwards, and the quantizers are deterministic, so the cached tensors are exactly what a fresh call
    would produce.  Valid while the parameters are the same tensors at the same version (``load_state_dict``,
    ``.to()``, in-place ops all change that; an edit through ``.data`` does not: call ``invalidate()``) and the
    quantizer settings passed as ``spec`` are the same.  Not used while gradients are recorded or a HIP graph is being
    captured."""

    def __init__(self):
        self.invalidate()

    def invalidate(self):
        self._key = None
        self.qw = self.qb = self._wb = self._wp = None

    @staticmethod
    def usable() -> bool:
        return not torch.is_grad_enabled() and not torch.cuda.is_current_stream_capturing()

    def get(self, weight: Tensor, bias: Tensor | None, spec, make):
        key = (_tensor_key(weight), _tensor_key(bias), spec)
        if key != self._key:
            self.invalidate()
            self.qw, self.qb = make()
            self._key = key
        return self.qw, self.qb

    def bf16(self) -> Tensor:
        if self._wb is None:
            self._wb = self.qw.to(torch.bfloat16).contiguous()
        return self._wb

    def packed(self):
        if self._wp is None and gemm_bf16_packed_b_supported(*self.qw.shape):
            self._wp = gemm_bf16_pack_b(self.bf16())
        return self._wp


def _quantized_params(cache, weight, bias, spec, quantize_weight, quantize_bias):
    """(quantized weight, quantized bias, cache or None): from ``cache`` when it may be used, else freshly computed"""
    make = lambda: (quantize_weight(weight), quantize_bias(bias) if bias is not None else None)
    if (cache is not None and weight.is_cuda and weight.dim() == 2 and QuantizedParamCache.usable()
            and _tensor_key(weight) is not None and _tensor_key(bias) is not None):  # None: an inference tensor
        qw, qb = cache.get(weight, bias, spec, make)
        return qw, qb, cache
    qw, qb = make()
    return qw, qb, None


def _contract(x: Tensor, weight: Tensor, bias: Tensor | None, exact_in_bf16: bool, cache=None) -> Tensor:
    """``F.linear(x, weight, bias)`` for already quantized operands.  The matrix-core kernel has no backward: it is
    used only when no gradient is being recorded (inference); training keeps the differentiable library GEMM.
    ``cache``: the ``QuantizedParamCache`` that holds ``weight``, for its bf16 and fragment-ordered copies."""
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad
                                              or (bias is not None and bias.requires_grad))
    if needs_grad or not (exact_in_bf16 and x.is_cuda and weight.dim() == 2 and x.numel() > 0
                          and x.dtype == weight.dtype and x.dtype in (torch.float32, torch.bfloat16, torch.float16)):
        return F.linear(x, weight, bias)
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1]).to(torch.bfloat16)
    if cache is not None:
        wp = cache.packed() if gemm_bf16_takes_packed_b(x2.shape[0], weight.shape[0], weight.shape[1]) else None
        y = gemm_bf16_tn(x2, cache.bf16(), bias, x.dtype, b_packed=wp)
    else:
        y = gemm_bf16_tn(x2, weight.to(torch.bfloat16), bias, x.dtype)
    return y.reshape(*lead, weight.shape[0])


def linearInteger(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None, out_config: dict = None, *,
                  param_cache: QuantizedParamCache | None = None):
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
    weight, bias, cache = _quantized_params(
        param_cache, weight, bias, ("integer", floor, w_width, w_frac_width, b_width, b_frac_width),
        lambda w: base_quantizer(w, width=w_width, frac_width=w_frac_width),
        lambda b: base_quantizer(b, width=b_width, frac_width=b_frac_width))
    out = _contract(x, weight, bias, max(w_width, x_width) <= 9, cache)
    if "data_out_width" in config or out_config is not None:
        out = base_quantizer(out, width=out_width, frac_width=out_frac_width)
    return out


def _linear_minifloat(quantizer, x, weight, bias, config, param_cache=None):
    wq = partial(quantizer, width=config["weight_width"], exponent_width=config["weight_exponent_width"],
                 exponent_bias=config["weight_exponent_bias"])
    xq = partial(quantizer, width=config["data_in_width"], exponent_width=config["data_in_exponent_width"],
                 exponent_bias=config["data_in_exponent_bias"])
    bq = partial(quantizer, width=config["bias_width"], exponent_width=config["bias_exponent_width"],
                 exponent_bias=config["bias_exponent_bias"])
    x = xq(x)
    spec = (quantizer.__name__, config["weight_width"], config["weight_exponent_width"], config["weight_exponent_bias"],
            config["bias_width"], config["bias_exponent_width"], config["bias_exponent_bias"])
    weight, bias, cache = _quantized_params(param_cache, weight, bias, spec, wq, bq)
    # mantissa bits (plus the implicit one of the ieee flavour) of both operands
    sig = max(config["weight_width"] - config["weight_exponent_width"] - 1,
              config["data_in_width"] - config["data_in_exponent_width"] - 1) + (1 if quantizer is minifloat_ieee_quantizer else 0)
    return _contract(x, weight, bias, sig <= 8, cache)


def linearMinifloatDenorm(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None, *,
                          param_cache: QuantizedParamCache | None = None):
    return _linear_minifloat(minifloat_denorm_quantizer, x, weight, bias, config, param_cache)


def linearMinifloatIEEE(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None, *,
                        param_cache: QuantizedParamCache | None = None):
    return _linear_minifloat(minifloat_ieee_quantizer, x, weight, bias, config, param_cache)


def linearBlockFP(x: Tensor, weight: Tensor, bias: Tensor = None, config: dict = None, *,
                  param_cache: QuantizedParamCache | None = None):
    w_cfg = (config["weight_width"], config["weight_exponent_width"], config["weight_exponent_bias"],
             config["weight_block_size"])
    x_cfg = (config["data_in_width"], config["data_in_exponent_width"], config["data_in_exponent_bias"],
             config["data_in_block_size"])
    x_skip_first_dim = config.get("data_in_skip_first_dim", True)
    b_cfg = (config["bias_width"], config["bias_exponent_width"], config["bias_exponent_bias"],
             config["bias_block_size"])
    x = block_fp_quantizer(x, *x_cfg, skip_first_dim=x_skip_first_dim)
    spec = ("block_fp",) + tuple(tuple(v) if isinstance(v, (list, tuple)) else v for v in w_cfg + b_cfg)
    weight, bias, cache = _quantized_params(
        param_cache, weight, bias, spec,
        lambda w: block_fp_quantizer(w, *w_cfg, skip_first_dim=False),
        lambda b: block_fp_quantizer(b, *b_cfg, skip_first_dim=False))
    return _contract(x, weight, bias, max(config["weight_width"], config["data_in_width"]) <= 9, cache)
