from .loader import DictSource, FolderSource, TensorSource, WeightError, check_tensors, load_model, load_weights
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors

__all__ = [
    "DictSource", "FolderSource", "TensorSource", "WeightError", "check_tensors", "load_model", "load_weights",
    "random_tensors", "write_random_model", "SafetensorsError", "SafetensorsFile", "open_model_files",
    "write_safetensors",
]
