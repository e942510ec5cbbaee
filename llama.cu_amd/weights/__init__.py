"""Weights: reading safetensors by tensor name, checking them against what the model's
parts expect, and writing a random model folder."""
from .safetensors_io import read_safetensors_header, open_safetensors, write_safetensors, SafetensorsError
from .loader import WeightError, load_weights, check_tensors
from .random import (fill_normal, random_tensors, register_initialiser, registered_initialisers, stream_key,
                     write_random_model)

__all__ = ["read_safetensors_header", "open_safetensors", "write_safetensors", "SafetensorsError", "WeightError",
           "load_weights", "check_tensors", "fill_normal", "random_tensors", "register_initialiser", "registered_initialisers",
           "stream_key", "write_random_model"]
