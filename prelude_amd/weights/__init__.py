from .loader import WeightError, check_tensors, load_into
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsFile, WeightFileError, WeightFiles, find_safetensor_files, write_safetensors

__all__ = ["WeightError", "check_tensors", "load_into", "random_tensors", "write_random_model", "SafetensorsFile",
           "WeightFileError", "WeightFiles", "find_safetensor_files", "write_safetensors"]
