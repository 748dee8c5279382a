"""Quantized modules and functional forms (drop-in for the in-scope part of ``chop.nn.quantized``)."""
from .functional import bmm_mxfp, bmm_mxint, matmul_mxfp, matmul_mxint, quantized_func_map  # noqa: F401
from .modules import (  # noqa: F401
    EmbeddingMXFP,
    EmbeddingMXInt,
    LinearBlockFP,
    LinearInteger,
    LinearMinifloatDenorm,
    LinearMinifloatIEEE,
    LinearMXFP,
    LinearMXInt,
    LlamaAttentionMXFP,
    LlamaAttentionMXInt,
    LlamaMLPMXFP,
    LlamaMLPMXInt,
    LlamaRMSNormMinifloat,
    Qwen3AttentionMXFP,
    Qwen3AttentionMXInt,
    Qwen3MLPMXFP,
    Qwen3MLPMXInt,
    Qwen3RMSNormMinifloat,
    quantized_module_map,
)
