"""Weights: safetensors reading and writing, the checked loader, seeded random weights."""
from .loader import WeightError, load_weights, target_dtype
from .random_init import random_tensor, random_weights, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, open_folder, save_file

__all__ = ["SafetensorsError", "SafetensorsFile", "WeightError", "load_weights", "open_folder",
           "random_tensor", "random_weights", "save_file", "target_dtype", "write_model_folder"]
