from .quantize import quantize_module_transform_pass  # noqa: F401
from .gptq import GPTQ, find_qlayers, gptq_decoder_layer, quantize_tensor, run_gptq  # noqa: F401
