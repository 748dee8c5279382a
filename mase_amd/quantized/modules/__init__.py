"""``quantized_module_map``: the in-scope entries of the reference's registry
(``chop/nn/quantized/modules/__init__.py:236-251, 334-335, 352-369, 388-408``), same keys."""
from .embedding import EmbeddingMXFP, EmbeddingMXInt
from .llama import (
    LlamaAttentionMXFP,
    LlamaAttentionMXInt,
    LlamaMLPMXFP,
    LlamaMLPMXInt,
    LlamaRMSNormMinifloat,
    quantized_llama_module_map,
)
from .qwen3 import (
    Qwen3AttentionMXFP,
    Qwen3AttentionMXInt,
    Qwen3MLPMXFP,
    Qwen3MLPMXInt,
    Qwen3RMSNormMinifloat,
    quantized_qwen3_module_map,
)
from .linear import (
    LinearBlockFP,
    LinearInteger,
    LinearMinifloatDenorm,
    LinearMinifloatIEEE,
    LinearMXFP,
    LinearMXInt,
)

quantized_module_map = {
    "linear_block_fp": LinearBlockFP,
    "linear_integer": LinearInteger,
    "linear_fixed": LinearInteger,
    "linear_minifloat_denorm": LinearMinifloatDenorm,
    "linear_minifloat_ieee": LinearMinifloatIEEE,
    "linear_mxint": LinearMXInt,
    "linear_mxfp": LinearMXFP,
    "embedding_mxint": EmbeddingMXInt,
    "embedding_mxfp": EmbeddingMXFP,
} | quantized_llama_module_map | quantized_qwen3_module_map
