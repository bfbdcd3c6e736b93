"""Weights: reading safetensors by tensor name, and random weights from a configuration and a seed."""
from .loader import WeightsError, load_weights, resolve_files, save_weights
from .random_init import init_tensor, random_tensors, write_random_model

__all__ = ["WeightsError", "load_weights", "resolve_files", "save_weights", "init_tensor", "random_tensors",
           "write_random_model"]
