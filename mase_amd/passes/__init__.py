from .quantize import quantize_module_transform_pass  # noqa: F401
from .gptq import InputGram, group_quantizer, round_decoder_layer, round_weight, run_gptq  # noqa: F401
