"""Weights: safetensors by tensor name, and the random-weights mode."""

from .loader import WeightsError, checkpoint_files, expected_tensors, load_weights
from .random_init import random_checkpoint_tensors, random_tensor, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, save_state_dict, write_safetensors

__all__ = [
    "SafetensorsError",
    "SafetensorsFile",
    "WeightsError",
    "checkpoint_files",
    "expected_tensors",
    "load_weights",
    "random_checkpoint_tensors",
    "random_tensor",
    "save_state_dict",
    "write_random_model",
    "write_safetensors",
]
