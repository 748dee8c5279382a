"""Quantized softmax / rotary embedding / SiLU / KV-cache functions with the names, config keys and behaviour of the
reference's ``chop/nn/quantized/functional/softmax.py:10-57``, ``rope.py:10-101``, ``silu.py:10-57`` and
``kvcache.py:8-43``: the input (for RoPE: the cos/sin tables) goes through an MXFP / MXINT / minifloat
quantize-dequantize (HIP kernels), the op itself is the ordinary torch one (softmax evaluated in fp32 and cast back).
"""
from __future__ import annotations

import torch
from torch import Tensor

from ...quantizers import mxfp_quantizer, mxint_quantizer
from ...quantizers import _ops
from ...quantizers._ops import minifloat_mx_qdq


def _q_mxfp(config):
    return lambda t: mxfp_quantizer(t, block_size=config["data_in_block_size"],
                                    element_exp_bits=config["data_in_exponent_width"],
                                    element_frac_bits=config["data_in_frac_width"], block_dim=-1)


def _q_mxint(config):
    return lambda t: mxint_quantizer(t, block_size=config["data_in_block_size"], element_bits=config["data_in_width"],
                                     block_dim=-1)


def _q_minifloat(config):
    """element-wise minifloat cast (``minifloat_quantizer_sim`` with a ``MinifloatMeta`` built from the config)"""
    return lambda t: minifloat_mx_qdq(t, config["data_in_exponent_width"], config["data_in_frac_width"],
                                      config.get("data_in_is_finite", True), config.get("data_in_round_mode", "rn"), None)


def _softmax(x: Tensor, dim: int) -> Tensor:
    return torch.nn.functional.softmax(x.to(torch.float32), dim=dim).to(x.dtype)


def softmax_mxfp(x: Tensor, config: dict = None, dim: int = -1) -> Tensor:
    return _softmax(_q_mxfp(config)(x), dim)


def softmax_mxint(x: Tensor, config: dict = None, dim: int = -1) -> Tensor:
    return _softmax(_q_mxint(config)(x), dim)


def softmax_minifloat(x: Tensor, config: dict = None, dim: int = -1) -> Tensor:
    return _softmax(_q_minifloat(config)(x), dim)


def silu_mxfp(x: Tensor, config: dict = None) -> Tensor:
    return torch.nn.functional.silu(_q_mxfp(config)(x))


def silu_mxint(x: Tensor, config: dict = None) -> Tensor:
    return torch.nn.functional.silu(_q_mxint(config)(x))


def silu_minifloat(x: Tensor, config: dict = None) -> Tensor:
    return torch.nn.functional.silu(_q_minifloat(config)(x))


def rotate_half(x: Tensor) -> Tensor:
    """Rotate half the last dimension (for RoPE)."""
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def _apply_rope(q, k, cos, sin, unsqueeze_dim=1):
    seq = q.size(-2)
    if unsqueeze_dim == 1 and cos.dim() == 3 and k.size(-2) == seq:  # one pass per tensor
        c, s_ = cos[..., :seq, :], sin[..., :seq, :]
        if _ops.rope_supported(q, c, s_) and _ops.rope_supported(k, c, s_):
            return _ops.rope(q, c, s_), _ops.rope(k, c, s_)
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    seq_len = q.size(-2)
    cos = cos[..., :seq_len, :]
    sin = sin[..., :seq_len, :]
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def rope_mxfp(q, k, cos, sin, config: dict = None, unsqueeze_dim: int = 1):
    qz = _q_mxfp(config)
    return _apply_rope(q, k, qz(cos), qz(sin), unsqueeze_dim)


def rope_mxint(q, k, cos, sin, config: dict = None, unsqueeze_dim: int = 1):
    qz = _q_mxint(config)
    return _apply_rope(q, k, qz(cos), qz(sin), unsqueeze_dim)


def rope_minifloat(q, k, cos, sin, config: dict = None, unsqueeze_dim: int = 1):
    qz = _q_minifloat(config)
    return _apply_rope(q, k, qz(cos), qz(sin), unsqueeze_dim)


def kv_cache_mxfp(key_states: Tensor, value_states: Tensor, config: dict = None):
    qz = _q_mxfp(config)
    return qz(key_states), qz(value_states)


def kv_cache_mxint(key_states: Tensor, value_states: Tensor, config: dict = None):
    qz = _q_mxint(config)
    return qz(key_states), qz(value_states)
