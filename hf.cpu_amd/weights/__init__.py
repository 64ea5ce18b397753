"""Weights: the safetensors container, loading by tensor name, random weights."""
from .loader import check_tensors, held_dtype, load_tensors
from .random_init import random_device_tensors, random_tensor, write_random_model
from .safetensors_io import SafetensorsFile, open_model_tensors, write_safetensors

__all__ = ["SafetensorsFile", "check_tensors", "held_dtype", "load_tensors", "open_model_tensors",
           "random_device_tensors", "random_tensor", "write_random_model", "write_safetensors"]
