"""Synthetic workloads used by the benchmark and the parity tests (not a model zoo)."""
from .decoder_layer import DecoderLayer, DecoderLayerConfig  # noqa: F401
