from .quantize import quantize_module_transform_pass  # noqa: F401
