"""MX-quantized Llama attention, MLP and RMSNorm with the constructor, attributes, config keys and forward contract
of the reference's ``chop/nn/quantized/modules/llama/attention.py:130-457`` (``LlamaAttentionMXFP``,
``LlamaAttentionMXInt``, ``_eager_attention_forward_mxfp/_mxint``), ``llama/mlp.py:49-77`` (``LlamaMLPMXFP``,
``LlamaMLPMXInt``) and ``llama/rms_norm.py:34-84`` (``LlamaRMSNormMinifloat``).

The reference derives these classes from the ``transformers`` Llama modules; here they are plain ``nn.Module``s with
the same parameter names (``q_proj/k_proj/v_proj/o_proj``, ``gate_proj/up_proj/down_proj``, ``weight``), so a state
dict of the original module loads with ``strict=True`` and no ``transformers`` import is needed.  ``config`` is any
object with the Llama config fields read below (a ``LlamaConfig`` works).  Every quantizer is a HIP kernel; the two
batched contractions (query x keys, probabilities x values: ``torch.matmul`` in the reference) run on the batched
matrix-core kernel of this package for bf16 operands (``mase_gemm_bf16_tn_batched``) and on ``torch.matmul`` otherwise.

What is quantized (``q_config`` sub-dicts, each with an optional ``bypass``):
  ``rope``      cos/sin tables, minifloat cast                       (attention.py:163-177)
  ``kv_cache``  new key/value states before ``past_key_value.update``  (attention.py:182-187)
  ``qk_matmul`` the query (not the key) along head_dim                (attention.py:352-361)
  ``softmax``   the masked scores, minifloat cast, softmax in fp32    (attention.py:369-375)
  ``av_matmul`` the probabilities (not the values) along the key axis (attention.py:383-392)
MLP: ``silu_minifloat`` on the gate projection (mlp.py:60-62, 75-77); RMSNorm: minifloat cast of the input and of the
weight (rms_norm.py:72-84).
"""
from __future__ import annotations

from functools import partial
from typing import Optional, Tuple

import torch
from torch import Tensor, nn

from ..._gemm import matmul_bf16
from ...quantizers import mxfp_quantizer, mxint_quantizer
from ...quantizers import _ops
from ...quantizers._ops import attn_softmax_mx, attn_softmax_mx_supported, minifloat_mx_qdq
from ..functional.mx_linear import project_shared
from ..functional.activations import kv_cache_mxfp, kv_cache_mxint, rope_minifloat, rotate_half, silu_minifloat, softmax_minifloat


def repeat_kv(hidden_states: Tensor, n_rep: int) -> Tensor:
    """(batch, kv_heads, seq, head_dim) -> (batch, kv_heads * n_rep, seq, head_dim), each head repeated in place"""
    batch, num_key_value_heads, slen, head_dim = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    hidden_states = hidden_states[:, :, None, :, :].expand(batch, num_key_value_heads, n_rep, slen, head_dim)
    return hidden_states.reshape(batch, num_key_value_heads * n_rep, slen, head_dim)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim=1):
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def _mx_quantizer(kind: str, config: dict):
    if kind == "mxfp":
        return partial(mxfp_quantizer, block_size=config["data_in_block_size"],
                       element_exp_bits=config["data_in_exponent_width"],
                       element_frac_bits=config["data_in_frac_width"], block_dim=-1)
    return partial(mxint_quantizer, block_size=config["data_in_block_size"], element_bits=config["data_in_width"],
                   block_dim=-1)


def _matmul(x, y, out=None):
    """``torch.matmul(x, y)``; bf16 device operands with equal leading dimensions run on the batched matrix-core kernel
    of this package (same arithmetic as the library's bf16 product: exact products, fp32 sums, one rounding)"""
    r = matmul_bf16(x, y, out=out) if x.is_cuda and x.dtype == torch.bfloat16 else None
    return torch.matmul(x, y) if r is None else r


def _value_product(probabilities, value_states):
    """``matmul(probabilities, value_states).transpose(1, 2).contiguous()``: [batch, tokens, heads, head_dim]; the own
    kernel writes that layout directly"""
    B, H, S, _ = probabilities.shape
    D = value_states.shape[-1]
    if probabilities.is_cuda and probabilities.dtype == torch.bfloat16 and (D * 2) % 16 == 0:
        out = torch.empty((B, S, H, D), dtype=probabilities.dtype, device=probabilities.device)
        if matmul_bf16(probabilities, value_states, out=out.transpose(1, 2)) is not None:
            return out
    return torch.matmul(probabilities, value_states).transpose(1, 2).contiguous()


def _eager_attention_forward(kind, module, query, key, value, attention_mask, scaling, dropout=0.0, qk_bypass=False,
                             qk_config=None, av_bypass=False, av_config=None, softmax_bypass=False, softmax_config=None,
                             **kwargs):
    key_states = repeat_kv(key, module.num_key_value_groups)
    value_states = repeat_kv(value, module.num_key_value_groups)
    if not qk_bypass:
        query = _mx_quantizer(kind, qk_config)(query)
    scores = _matmul(query, key_states.transpose(2, 3))
    fused = _fused_probabilities(kind, module, scores, key_states, attention_mask, scaling, dropout, av_bypass, av_config,
                                 softmax_bypass, softmax_config)
    if fused is not None:
        return _value_product(fused, value_states), fused
    attn_weights = scores * scaling
    if attention_mask is not None:
        causal_mask = attention_mask[:, :, :, : key_states.shape[-2]]
        attn_weights = attn_weights + causal_mask
    if not softmax_bypass:
        attn_weights = softmax_minifloat(attn_weights, softmax_config, dim=-1)
    else:
        attn_weights = nn.functional.softmax(attn_weights.to(torch.float32), dim=-1).to(attn_weights.dtype)
    attn_weights = nn.functional.dropout(attn_weights, p=dropout, training=module.training)
    if not av_bypass:
        attn_weights = _mx_quantizer(kind, av_config)(attn_weights)
    return _value_product(attn_weights, value_states), attn_weights


def _fused_probabilities(kind, module, scores, key_states, attention_mask, scaling, dropout, av_bypass, av_config,
                         softmax_bypass, softmax_config):
    """scores -> scaled, masked, minifloat-cast, softmax, MX-quantized probabilities in one kernel when the operands
    allow it (device tensors, key length a multiple of 32 up to 8192, blocks of 32, no dropout); else None and the
    caller runs the separate passes.  Opt-in (``module.fused_probabilities = True``): the kernel evaluates the
    exponentials with the hardware ``exp2`` and about one probability in a hundred lands on the neighbouring code, while
    the separate passes are the reference's own tensor operations on the device."""
    if not getattr(module, "fused_probabilities", False) or not scores.is_cuda:
        return None
    if dropout != 0.0 and module.training:
        return None
    if torch.is_grad_enabled() and scores.requires_grad:
        return None
    mx = None
    if not av_bypass:
        if av_config["data_in_block_size"] != 32:
            return None
        mx = ("mxfp", av_config["data_in_exponent_width"], av_config["data_in_frac_width"]) if kind == "mxfp" \
            else ("mxint", av_config["data_in_width"])
    cast = None
    if not softmax_bypass:
        cast = (softmax_config["data_in_exponent_width"], softmax_config["data_in_frac_width"],
                softmax_config.get("data_in_is_finite", True), softmax_config.get("data_in_round_mode", "rn"))
    mask = None
    if attention_mask is not None:
        mask = attention_mask[:, :, :, : key_states.shape[-2]]
    if not attn_softmax_mx_supported(scores, mask):
        return None
    return attn_softmax_mx(scores, mask, scaling, cast, mx)


_eager_attention_forward_mxfp = partial(_eager_attention_forward, "mxfp")
_eager_attention_forward_mxint = partial(_eager_attention_forward, "mxint")


class _LlamaAttentionMX(nn.Module):
    _kind = "mxint"

    def __init__(self, config, layer_idx, q_config: dict = None):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads
        self.scaling = self.head_dim ** -0.5
        self.attention_dropout = getattr(config, "attention_dropout", 0.0)
        self.is_causal = True
        bias = getattr(config, "attention_bias", False)
        self.q_proj = nn.Linear(config.hidden_size, config.num_attention_heads * self.head_dim, bias=bias)
        self.k_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.v_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.o_proj = nn.Linear(config.num_attention_heads * self.head_dim, config.hidden_size, bias=bias)
        q_config = q_config or {}
        self.qk_config = q_config.get("qk_matmul", {})
        self.av_config = q_config.get("av_matmul", {})
        self.rope_config = q_config.get("rope", {})
        self.softmax_config = q_config.get("softmax", {})
        self.kv_cache_config = q_config.get("kv_cache", {})
        self.qk_bypass = self.qk_config.get("bypass", False)
        self.av_bypass = self.av_config.get("bypass", False)
        self.rope_bypass = self.rope_config.get("bypass", False)
        self.softmax_bypass = self.softmax_config.get("bypass", False)
        self.kv_cache_bypass = self.kv_cache_config.get("bypass", False)

    def forward(self, hidden_states: Tensor, position_embeddings: Tuple[Tensor, Tensor],
                attention_mask: Optional[Tensor], past_key_value=None, cache_position=None, **kwargs):
        input_shape = hidden_states.shape[:-1]
        hidden_shape = (*input_shape, -1, self.head_dim)
        query_states, key_states, value_states = self._project(hidden_states, hidden_shape)

        cos, sin = position_embeddings
        if not self.rope_bypass:
            query_states, key_states = rope_minifloat(query_states, key_states, cos, sin, self.rope_config)
        else:
            query_states, key_states = apply_rotary_pos_emb(query_states, key_states, cos, sin)

        if past_key_value is not None:
            cache_kwargs = {"sin": sin, "cos": cos, "cache_position": cache_position}
            if not self.kv_cache_bypass:
                kv_cache = kv_cache_mxfp if self._kind == "mxfp" else kv_cache_mxint
                key_states, value_states = kv_cache(key_states, value_states, self.kv_cache_config)
            key_states, value_states = past_key_value.update(key_states, value_states, self.layer_idx, cache_kwargs)

        attn_output, attn_weights = _eager_attention_forward(
            self._kind, self, query_states, key_states, value_states, attention_mask,
            dropout=0.0 if not self.training else self.attention_dropout, scaling=self.scaling,
            qk_bypass=self.qk_bypass, qk_config=self.qk_config, av_bypass=self.av_bypass, av_config=self.av_config,
            softmax_bypass=self.softmax_bypass, softmax_config=self.softmax_config, **kwargs)
        attn_output = attn_output.reshape(*input_shape, -1).contiguous()
        attn_output = self.o_proj(attn_output)
        return attn_output, attn_weights

    def _project(self, hidden_states, hidden_shape):
        """query / key / value states [batch, heads, seq, head_dim] (attention.py:157-159)"""
        q, k, v = project_shared(hidden_states, (self.q_proj, self.k_proj, self.v_proj))
        return tuple(t.view(hidden_shape).transpose(1, 2) for t in (q, k, v))

    @classmethod
    def from_attention(cls, attention: nn.Module, q_config: dict = None):
        new_attn = cls(config=attention.config, layer_idx=attention.layer_idx, q_config=q_config)
        first = next(attention.parameters())
        new_attn = new_attn.to(dtype=first.dtype, device=first.device)
        new_attn.load_state_dict(attention.state_dict(), strict=True)
        return new_attn


class LlamaAttentionMXFP(_LlamaAttentionMX):
    """MXFP-quantized Llama attention."""
    _kind = "mxfp"


class LlamaAttentionMXInt(_LlamaAttentionMX):
    """MXInt-quantized Llama attention."""
    _kind = "mxint"


class _LlamaMLPMX(nn.Module):
    """Llama MLP whose SiLU input goes through the minifloat cast."""

    def __init__(self, config, layer_idx=None, q_config: dict = None):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        bias = getattr(config, "mlp_bias", False)
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=bias)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=bias)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=bias)
        hidden_act = getattr(config, "hidden_act", "silu")
        if hidden_act != "silu":
            raise NotImplementedError(f"hidden_act={hidden_act!r}: the quantized form is defined for SiLU only")
        self.act_fn = nn.SiLU()
        self.layer_idx = layer_idx
        self.q_config = q_config or {}
        self.bypass = self.q_config.get("bypass", False)

    def forward(self, x: Tensor) -> Tensor:
        gate, up = project_shared(x, (self.gate_proj, self.up_proj))
        if _ops.silu_mul_supported(gate, up):  # one pass: cast, SiLU and product
            cast = None if self.bypass else (self.q_config["data_in_exponent_width"], self.q_config["data_in_frac_width"],
                                             self.q_config.get("data_in_is_finite", True),
                                             self.q_config.get("data_in_round_mode", "rn"))
            return self.down_proj(_ops.silu_mul_minifloat(gate, up, cast))
        if self.bypass:
            return self.down_proj(self.act_fn(gate) * up)
        return self.down_proj(silu_minifloat(gate, self.q_config) * up)


class LlamaMLPMXFP(_LlamaMLPMX):
    """MXFP-quantized LlamaMLP. SiLU uses minifloat quantization."""


class LlamaMLPMXInt(_LlamaMLPMX):
    """MXInt-quantized LlamaMLP. SiLU uses minifloat quantization."""


class LlamaRMSNormMinifloat(nn.Module):
    """Minifloat-quantized Llama RMSNorm: weight and input go through the minifloat cast at forward time."""

    def __init__(self, config=None, layer_idx=None, q_config: dict = None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(config.hidden_size))
        self.variance_epsilon = config.rms_norm_eps
        self.layer_idx = layer_idx
        self.q_config = q_config or {}
        self.bypass = self.q_config.get("bypass", False)
        self.weight_bypass = self.q_config.get("weight_bypass", False)
        self.data_in_bypass = self.q_config.get("data_in_bypass", False)

        def cast(prefix):
            return partial(minifloat_mx_qdq, exp_bits=self.q_config[f"{prefix}_exponent_width"],
                           frac_bits=self.q_config[f"{prefix}_frac_width"],
                           is_finite=self.q_config.get(f"{prefix}_is_finite", True),
                           round_mode=self.q_config.get(f"{prefix}_round_mode", "rn"), output_dtype=None)

        self.w_quantizer = cast("weight") if not self.bypass and not self.weight_bypass else None
        self.x_quantizer = cast("data_in") if not self.bypass and not self.data_in_bypass else None

    def _cast_spec(self, prefix, quantizer):
        if quantizer is None:
            return None
        return (self.q_config[f"{prefix}_exponent_width"], self.q_config[f"{prefix}_frac_width"],
                self.q_config.get(f"{prefix}_is_finite", True), self.q_config.get(f"{prefix}_round_mode", "rn"))

    def forward(self, hidden_states):
        if _ops.rmsnorm_supported(hidden_states, self.weight):  # one pass over the activations
            return _ops.rmsnorm_minifloat(hidden_states, self.weight, self.variance_epsilon,
                                          self._cast_spec("data_in", self.x_quantizer),
                                          self._cast_spec("weight", self.w_quantizer))
        input_dtype = hidden_states.dtype
        if self.x_quantizer is not None:
            hidden_states = self.x_quantizer(hidden_states)
        hidden_states = hidden_states.to(torch.float32)
        variance = hidden_states.pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        weight = self.w_quantizer(self.weight) if self.w_quantizer is not None else self.weight
        return weight * hidden_states.to(input_dtype)

    def extra_repr(self):
        return f"{tuple(self.weight.shape)}, eps={self.variance_epsilon}"


quantized_llama_module_map = {
    "llama_self_attention_mxfp": LlamaAttentionMXFP,
    "llama_self_attention_mxint": LlamaAttentionMXInt,
    "llama_rms_norm_minifloat": LlamaRMSNormMinifloat,
    "llama_mlp_mxfp": LlamaMLPMXFP,
    "llama_mlp_mxint": LlamaMLPMXInt,
}
