"""Weights: the safetensors container, binding by name, random weights."""
from .loader import WeightError, check_names_and_shapes, load_tensors, storage_dtype
from .random_init import random_tensors, write_model_folder
from .safetensors_io import SafetensorsFile, WeightFileError, open_model_files, write_safetensors

__all__ = [
    "WeightError", "check_names_and_shapes", "load_tensors", "storage_dtype", "random_tensors",
    "write_model_folder", "SafetensorsFile", "WeightFileError", "open_model_files", "write_safetensors",
]
