"""Weights: reading safetensors by tensor name, checking them against what a
model expects, placing them on the device; and writing random model folders."""

from .loader import WeightError, place_tensors, read_safetensors
from .random_init import write_model_folder

__all__ = ["WeightError", "place_tensors", "read_safetensors", "write_model_folder"]
