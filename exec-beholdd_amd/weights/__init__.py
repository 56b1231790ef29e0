"""Checkpoints: the safetensors reader and writer, binding by name, seeded random weights."""

from .binder import BoundWeights, TensorSpec, WeightError, bind, check_manifest, stored_dtype
from .random_init import random_tensor, random_tensor_on_device, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsReader, write_safetensors

__all__ = ["BoundWeights", "TensorSpec", "WeightError", "bind", "check_manifest", "stored_dtype",
           "random_tensor", "random_tensor_on_device", "write_random_model", "SafetensorsError",
           "SafetensorsReader", "write_safetensors"]
