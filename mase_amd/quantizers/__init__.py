"""Drop-in for the in-scope part of the reference's ``chop.nn.quantizers`` (``__init__.py:1-28``).

Same function names, argument order, defaults and straight-through gradients; the forward arithmetic runs
in hand-written gfx950 kernels.  Tensors must live on a ROCm device.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

import torch
from torch import Tensor

from . import _ops


class _STE(torch.autograd.Function):
    """Straight-through estimator shared by all quantizers: backward is ``grad_output.clone()``
    (reference: mxint/mxint.py:204-208, block_fp.py:105-108, integer.py:78-81)."""

    @staticmethod
    def forward(ctx, x, fn, args):
        return fn(x, *args)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output.clone(), None, None


def _ste(fn, x: Tensor, *args):
    if x.requires_grad and torch.is_grad_enabled():
        return _STE.apply(x, fn, args)
    return fn(x, *args)


# ---------------------------------------------------------------------------------------------
# metadata classes (mxint/meta.py:8-34, mxfp/meta.py:12-67, _minifloat_mx/meta.py:10-42)
# ---------------------------------------------------------------------------------------------
@dataclass
class MXIntMeta:
    block_size: int
    scale_bits: int
    element_bits: int


@dataclass(frozen=True)
class MinifloatMeta:
    exp_bits: int
    frac_bits: int
    is_finite: bool
    round_mode: Literal["rn", "rd", "ru", "rz"]

    def __post_init__(self):
        assert self.exp_bits > 0
        assert self.frac_bits > 0
        assert self.exp_bits + self.frac_bits < 16

    @property
    def n_bits(self) -> int:
        return self.exp_bits + self.frac_bits + 1


@dataclass(frozen=True)
class MXFPMeta:
    block_size: int
    scale_exp_bits: int
    element_exp_bits: int
    element_frac_bits: int
    element_is_finite: bool
    round_mode: Literal["rn", "ru", "rd", "rz"]

    def __post_init__(self):
        legal_scale_exp_bits = (8,)
        assert self.scale_exp_bits in legal_scale_exp_bits, (
            f"Invalid scale exponent bits: {self.scale_exp_bits}. Legal values are: {legal_scale_exp_bits}."
        )
        el = (self.element_exp_bits, self.element_frac_bits)
        assert el in _ops._LEGAL_MXFP, f"Invalid element exp/frac bits: {el}. Legal values are: {_ops._LEGAL_MXFP}."

    @property
    def element_meta(self) -> MinifloatMeta:
        return MinifloatMeta(self.element_exp_bits, self.element_frac_bits, self.element_is_finite, self.round_mode)


# ---------------------------------------------------------------------------------------------
# MXINT
# ---------------------------------------------------------------------------------------------
def mxint_quantizer_sim(tensor: Tensor, block_dim: int, mxint_meta: MXIntMeta, act_tensor: Tensor | None = None,
                        dtype: torch.dtype | None = None, quantile_search: bool = False,
                        cali_batch_size: int = 32) -> Tensor:
    """mxint/mxint.py:14-171, both forms of the search branch (:40-143): scored on the weights themselves, or with
    ``act_tensor`` [batches, tokens, block_size] on the products with calibration activations."""
    if quantile_search:
        if act_tensor is not None:
            return _ops.mxint_clip_search_calibrated(tensor, mxint_meta.block_size, mxint_meta.element_bits, block_dim,
                                                     mxint_meta.scale_bits, act_tensor, cali_batch_size)
        return _ops.mxint_clip_search(tensor, mxint_meta.block_size, mxint_meta.element_bits, block_dim,
                                      mxint_meta.scale_bits)  # the search branch ignores `dtype` (mxint.py:143)
    out = _ops.mxint_qdq(tensor, mxint_meta.block_size, mxint_meta.element_bits, block_dim, mxint_meta.scale_bits)
    return out.to(dtype or tensor.dtype)


def mxint_quantizer(x: Tensor, block_size: int, element_bits: int, block_dim: int = -1, scale_bits: int = 8,
                    quantile_search: bool = False) -> Tensor:
    """MXINT quantize-dequantize with a straight-through gradient (mxint/mxint.py:211-251)."""
    if quantile_search:
        return _ste(_ops.mxint_clip_search, x, block_size, element_bits, block_dim, scale_bits)
    return _ste(_ops.mxint_qdq, x, block_size, element_bits, block_dim, scale_bits)


# ---------------------------------------------------------------------------------------------
# MXFP and the bit-level minifloat cast
# ---------------------------------------------------------------------------------------------
def minifloat_quantizer_sim(tensor: Tensor, minifloat_meta: MinifloatMeta,
                            output_dtype: torch.dtype | None = None) -> Tensor:
    """_minifloat_mx/minifloat.py:12-33."""
    return _ops.minifloat_mx_qdq(tensor, minifloat_meta.exp_bits, minifloat_meta.frac_bits, minifloat_meta.is_finite,
                                 minifloat_meta.round_mode, output_dtype)


def mxfp_quantizer_sim(tensor: Tensor, block_dim: int, mxfp_meta: MXFPMeta, act_tensor: Tensor | None = None,
                       dtype: torch.dtype | None = None, quantile_search: bool = False,
                       cali_batch_size: int = 32) -> Tensor:
    """mxfp/mxfp.py:14-115 (finite elements, round-to-nearest as MXFPQuantize fixes them); the search branch
    (:40-105) scored on the weights themselves or, with ``act_tensor`` [batches, tokens, block_size], on the products
    with calibration activations."""
    if not (mxfp_meta.element_is_finite and mxfp_meta.round_mode == "rn"):
        raise NotImplementedError("mxfp_quantizer_sim: only finite elements with round mode 'rn' are accelerated")
    if quantile_search:
        if act_tensor is not None:
            out = _ops.mxfp_clip_search_calibrated(tensor, mxfp_meta.block_size, mxfp_meta.element_exp_bits,
                                                   mxfp_meta.element_frac_bits, block_dim, mxfp_meta.scale_exp_bits,
                                                   act_tensor, cali_batch_size)
            return out.to(dtype or tensor.dtype)
        out = _ops.mxfp_clip_search(tensor, mxfp_meta.block_size, mxfp_meta.element_exp_bits,
                                    mxfp_meta.element_frac_bits, block_dim, mxfp_meta.scale_exp_bits)
        return out.to(dtype or tensor.dtype)
    out = _ops.mxfp_qdq(tensor, mxfp_meta.block_size, mxfp_meta.element_exp_bits, mxfp_meta.element_frac_bits,
                        block_dim, mxfp_meta.scale_exp_bits)
    return out.to(dtype or tensor.dtype)


def mxfp_quantizer(x: Tensor, block_size: int, element_exp_bits: int, element_frac_bits: int, block_dim: int = -1,
                   scale_exp_bits: int = 8, quantile_search: bool = False) -> Tensor:
    """MXFP quantize-dequantize with a straight-through gradient (mxfp/mxfp.py:187-230)."""
    if quantile_search:
        return _ste(_ops.mxfp_clip_search, x, block_size, element_exp_bits, element_frac_bits, block_dim, scale_exp_bits)
    return _ste(_ops.mxfp_qdq, x, block_size, element_exp_bits, element_frac_bits, block_dim, scale_exp_bits)


# ---------------------------------------------------------------------------------------------
# block floating point, fixed point, element-wise minifloat
# ---------------------------------------------------------------------------------------------
def block_fp_quantizer(x: Tensor, width: int = 12, exponent_width: int = 8, exponent_bias: int = None,
                       block_size: list[int] = [16], skip_first_dim: bool = True):
    """Block floating point (MSFP) quantize-dequantize (block_fp.py:111-142)."""
    return _ste(_ops.block_fp_qdq, x, width, exponent_width, exponent_bias, block_size, skip_first_dim)


def integer_quantizer(x: Tensor, width: int, frac_width: int, is_signed: bool = True):
    """Fixed-point quantize-dequantize, round half to even (integer.py:97-116)."""
    if isinstance(x, int):
        return x
    return _ste(_ops.integer_qdq, x, width, frac_width, is_signed, False)


def integer_floor_quantizer(x: Tensor, width: int, frac_width: int, is_signed: bool = True):
    """Fixed-point quantize-dequantize with floor (integer.py:119-122)."""
    if isinstance(x, int):
        return x
    return _ste(_ops.integer_qdq, x, width, frac_width, is_signed, True)


def minifloat_denorm_quantizer(x: Tensor, width: int, exponent_width: int, exponent_bias: int = None):
    """Minifloat without implicit leading bit (minifloat.py:90-117)."""
    return _ste(_ops.minifloat_qdq, x, width, exponent_width, exponent_bias, False)


def minifloat_ieee_quantizer(x: Tensor, width: int, exponent_width: int, exponent_bias: int = None):
    """Minifloat with implicit leading bit (minifloat.py:200-225)."""
    return _ste(_ops.minifloat_qdq, x, width, exponent_width, exponent_bias, True)


# the in-scope entries of the reference's registry (__init__.py:14-28)
quantizer_map = {
    "minifloat_denorm": minifloat_denorm_quantizer,
    "minifloat_ieee": minifloat_ieee_quantizer,
    "block_fp": block_fp_quantizer,
    "integer": integer_quantizer,
    "mxfp": mxfp_quantizer,
    "mxint": mxint_quantizer,
}

__all__ = [
    "MXIntMeta", "MXFPMeta", "MinifloatMeta",
    "mxint_quantizer", "mxint_quantizer_sim", "mxfp_quantizer", "mxfp_quantizer_sim", "minifloat_quantizer_sim",
    "block_fp_quantizer", "integer_quantizer", "integer_floor_quantizer",
    "minifloat_denorm_quantizer", "minifloat_ieee_quantizer", "quantizer_map",
]
