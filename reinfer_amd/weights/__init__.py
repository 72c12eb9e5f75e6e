from .loader import (INT_TABLE, MATRIX, VECTOR, ParamDecl, WeightError, check_tensors, load_weights,
                     storage_dtype, weight_from_folder)
from .random_init import random_tensor, random_tensors, splitmix64, tensor_seed, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = [
    "INT_TABLE", "MATRIX", "VECTOR", "ParamDecl", "WeightError", "check_tensors", "load_weights",
    "storage_dtype", "weight_from_folder", "random_tensor", "random_tensors", "splitmix64", "tensor_seed", "write_model_folder",
    "SafetensorsError", "SafetensorsFile", "write_safetensors",
]
