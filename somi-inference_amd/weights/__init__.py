"""Weights by tensor name: file format, sources, validation, random mode."""

from .loader import WeightFetcher, WeightMismatchError, check_weights, device_dtype
from .random_init import write_random_model
from .safetensors_io import SafetensorsError, read_header, read_tensor, write_file
from .source import RandomSource, SafetensorsSource, WeightSource, random_tensor, tensor_seed
from .spec import MATRIX, TABLE, VECTOR, Init, WeightSpec

__all__ = [
    "Init", "MATRIX", "RandomSource", "SafetensorsError", "SafetensorsSource", "TABLE", "VECTOR",
    "WeightFetcher", "WeightMismatchError", "WeightSource", "WeightSpec", "check_weights",
    "device_dtype", "random_tensor", "read_header", "read_tensor", "tensor_seed", "write_file",
    "write_random_model",
]
