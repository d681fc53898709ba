"""Weights: the safetensors container, the strict loader and the random-weights mode."""

from .loader import CheckpointError, load_model, parse_dtype
from .random_init import write_random_model
from .safetensors_io import SafetensorsFile, SafetensorsFormatError, write_safetensors

__all__ = ["CheckpointError", "SafetensorsFile", "SafetensorsFormatError", "load_model", "parse_dtype",
           "write_random_model", "write_safetensors"]
