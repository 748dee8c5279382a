from .linear import linearBlockFP, linearInteger, linearMinifloatDenorm, linearMinifloatIEEE  # noqa: F401
from .mx_linear import mx_linear  # noqa: F401
from .matmul import bmm_mxfp, bmm_mxint, matmul_mxfp, matmul_mxint, quantized_func_map  # noqa: F401
from .activations import (  # noqa: F401
    kv_cache_mxfp,
    kv_cache_mxint,
    rope_minifloat,
    rope_mxfp,
    rope_mxint,
    silu_minifloat,
    silu_mxfp,
    silu_mxint,
    softmax_minifloat,
    softmax_mxfp,
    softmax_mxint,
)
