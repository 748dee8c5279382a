from .linear import linearBlockFP, linearInteger, linearMinifloatDenorm, linearMinifloatIEEE  # noqa: F401
from .mx_linear import mx_linear  # noqa: F401
from .matmul import bmm_mxfp, bmm_mxint, matmul_mxfp, matmul_mxint, quantized_func_map  # noqa: F401
