"""MX-quantized Qwen3 attention, MLP and RMSNorm with the contract of the reference's
``chop/nn/quantized/modules/qwen3/attention.py:23-361`` (``Qwen3AttentionMXFP``, ``Qwen3AttentionMXInt``),
``qwen3/mlp.py:8-37`` (``Qwen3MLPMXFP``, ``Qwen3MLPMXInt``) and ``qwen3/rms_norm.py:11-61`` (``Qwen3RMSNormMinifloat``).

Qwen3 differs from Llama in one step: the query and key projections go through an RMSNorm over ``head_dim``
(``q_norm`` / ``k_norm``, attention.py:53-59) before the rotary embedding.  Everything else (what is quantized and
where, the config keys, the one-pass score -> probability kernel) is the Llama module of this package.  As there, the
classes are plain ``nn.Module``s with the parameter names of the ``transformers`` modules, so their state dicts load
with ``strict=True``.
"""
from __future__ import annotations

import torch
from torch import nn

from ..functional.mx_linear import project_shared
from .llama import LlamaRMSNormMinifloat, _LlamaAttentionMX, _LlamaMLPMX


class _HeadRMSNorm(nn.Module):
    """RMSNorm over the last dimension with a learned weight (the ``transformers`` Qwen3RMSNorm arithmetic: fp32
    statistics, result cast back, then the weight)"""

    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        input_dtype = hidden_states.dtype
        hidden_states = hidden_states.to(torch.float32)
        variance = hidden_states.pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        return self.weight * hidden_states.to(input_dtype)


class _Qwen3AttentionMX(_LlamaAttentionMX):
    def __init__(self, config, layer_idx, q_config: dict = None):
        super().__init__(config, layer_idx, q_config)
        self.q_norm = _HeadRMSNorm(self.head_dim, config.rms_norm_eps)
        self.k_norm = _HeadRMSNorm(self.head_dim, config.rms_norm_eps)

    def _project(self, hidden_states, hidden_shape):
        q, k, v = project_shared(hidden_states, (self.q_proj, self.k_proj, self.v_proj))
        query_states = self.q_norm(q.view(hidden_shape)).transpose(1, 2)
        key_states = self.k_norm(k.view(hidden_shape)).transpose(1, 2)
        return query_states, key_states, v.view(hidden_shape).transpose(1, 2)


class Qwen3AttentionMXFP(_Qwen3AttentionMX):
    """MXFP-quantized Qwen3 attention."""
    _kind = "mxfp"


class Qwen3AttentionMXInt(_Qwen3AttentionMX):
    """MXInt-quantized Qwen3 attention."""
    _kind = "mxint"


class Qwen3MLPMXFP(_LlamaMLPMX):
    """MXFP-quantized Qwen3 MLP: the SiLU input goes through the minifloat cast."""


class Qwen3MLPMXInt(_LlamaMLPMX):
    """MXInt-quantized Qwen3 MLP: the SiLU input goes through the minifloat cast."""


class Qwen3RMSNormMinifloat(LlamaRMSNormMinifloat):
    """Qwen3 RMSNorm with minifloat casts of the input and the weight."""


quantized_qwen3_module_map = {
    "qwen3_self_attention_mxfp": Qwen3AttentionMXFP,
    "qwen3_self_attention_mxint": Qwen3AttentionMXInt,
    "qwen3_rms_norm_minifloat": Qwen3RMSNormMinifloat,
    "qwen3_mlp_mxfp": Qwen3MLPMXFP,
    "qwen3_mlp_mxint": Qwen3MLPMXInt,
}
