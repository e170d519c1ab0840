"""Weights: safetensors by tensor name, the loader with its one error, random weights."""

from .loader import (DictSource, FolderSource, WeightLoadError, check_source, load_model_folder,
                     load_weights)
from .random_init import RandomSource, random_state, write_random_model
from .safetensors_io import SafetensorsFile, save_file, weight_files

__all__ = [
    "DictSource", "FolderSource", "SafetensorsFile", "WeightLoadError", "check_source",
    "RandomSource", "load_model_folder", "load_weights", "random_state", "save_file", "weight_files",
    "write_random_model",
]
