"""Weights: the safetensors format, binding by name, random weights."""
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .loader import CheckpointSource, WeightError, check_names, load_tensors
from .random_init import RandomSource, make_tensor, random_tensors, write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "write_safetensors", "WeightError",
           "check_names", "load_tensors", "CheckpointSource", "RandomSource", "make_tensor", "random_tensors",
           "write_random_model"]
