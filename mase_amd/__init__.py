"""mase_amd: MI355X (gfx950) kernels behind MASE's quantizer and quantized-Linear interfaces.

``mase_amd.quantizers``          drop-in for ``chop.nn.quantizers`` (mxint, mxfp, block_fp, integer, minifloat)
``mase_amd.quantized``           drop-in for the quantized ``Linear`` modules and ``quantized_module_map``
``mase_amd.passes``              a minimal ``quantize_module_transform_pass`` with the reference's contract
"""
__version__ = "0.1.0"
