"""Quantized modules and functional forms (drop-in for the in-scope part of ``chop.nn.quantized``)."""
from .modules import (  # noqa: F401
    LinearBlockFP,
    LinearInteger,
    LinearMinifloatDenorm,
    LinearMinifloatIEEE,
    LinearMXFP,
    LinearMXInt,
    quantized_module_map,
)
