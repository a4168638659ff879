"""Checkpoints: safetensors reading and writing, binding by tensor name, random weights."""
from .loader import Checkpoint, WeightsError, check_checkpoint, device_dtype_of, expected_tensors, load_into
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Checkpoint", "WeightsError", "check_checkpoint", "device_dtype_of", "expected_tensors", "load_into",
           "random_tensor", "random_tensors", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "write_safetensors"]
