"""Checkpoint files, the loader that binds them to a model by tensor name, and random weights."""
from .safetensors_io import ModelFiles, SafetensorsError, SafetensorsFile, write_safetensors
from .loader import WeightError, Weights, check_names, load_weights, random_weights
from .random_init import random_tensors, write_random_model

__all__ = ["ModelFiles", "SafetensorsError", "SafetensorsFile", "write_safetensors", "WeightError", "Weights",
           "check_names", "load_weights", "random_weights", "random_tensors", "write_random_model"]
