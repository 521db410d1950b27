from .loader import WeightsError, bind_tensors, check_names, load_weights
from .random_init import random_tensors, write_model_dir
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .spec import INT_TABLE, MATRIX, TABLE, VECTOR, Normal, TensorSpec

__all__ = [
    "INT_TABLE", "MATRIX", "TABLE", "VECTOR", "Normal", "TensorSpec",
    "SafetensorsError", "SafetensorsFile", "write_safetensors",
    "WeightsError", "bind_tensors", "check_names", "load_weights",
    "random_tensors", "write_model_dir",
]
