"""Weights: safetensors by tensor name, and seeded random weights."""

from .loader import WeightError, check_folder, index_folder, load_tensors
from .random import INITIALIZERS, random_tensor, random_tensors, register_initializer, write_random_model

__all__ = ["WeightError", "check_folder", "index_folder", "load_tensors", "random_tensor", "random_tensors",
           "write_random_model", "INITIALIZERS", "register_initializer"]
