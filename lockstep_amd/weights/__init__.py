"""Weights: safetensors by tensor name, checks, and the random-weights mode."""

from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_tensors, save_file
from .store import (WeightError, WeightStore, check_names_and_shapes, load_weights, normalise_dtype,
                    weights_from_dict)

__all__ = ["random_tensors", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "open_model_tensors", "save_file", "WeightError", "WeightStore", "check_names_and_shapes",
           "load_weights", "normalise_dtype", "weights_from_dict"]
