from .loader import WeightError, check_tensors, load_into
from .random_init import load_random, random_tensors, random_tensors_on_device, write_random_model
from .safetensors_io import SafetensorsFile, WeightFileError, WeightFiles, find_safetensor_files, write_safetensors

__all__ = ["WeightError", "check_tensors", "load_into", "load_random", "random_tensors", "random_tensors_on_device", "write_random_model", "SafetensorsFile",
           "WeightFileError", "WeightFiles", "find_safetensor_files", "write_safetensors"]
