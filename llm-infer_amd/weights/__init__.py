from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .loader import ParamSpec, WeightError, read_checkpoint, check_tensors, place_tensor, load_into
from .random_init import random_tensors, write_random_model

__all__ = ["SafetensorsFile", "SafetensorsError", "write_safetensors", "ParamSpec", "WeightError",
           "read_checkpoint", "check_tensors", "place_tensor", "load_into", "random_tensors",
           "write_random_model"]
