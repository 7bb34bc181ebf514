"""Weights: the safetensors format, binding by name, random weights."""
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .loader import WeightError, check_names, load_tensors
from .random_init import random_tensors, write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "write_safetensors", "WeightError",
           "check_names", "load_tensors", "random_tensors", "write_random_model"]
