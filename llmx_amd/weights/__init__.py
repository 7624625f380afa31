"""Weights: safetensors by tensor name, and seeded random weights."""

from .loader import ModelFiles, WeightsError, check, device_dtype, load
from .random_init import RandomInit, host_values, stored_dtype, tensor_key
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["ModelFiles", "WeightsError", "check", "device_dtype", "load", "RandomInit", "host_values", "stored_dtype", "tensor_key",
           "SafetensorsError", "SafetensorsFile", "write_safetensors"]
