from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .gguf_io import GGUFFile, GGUFError, write_gguf
from .loader import ParamSpec, WeightError, OnDemand, read_checkpoint, check_tensors, place_tensor, load_into, choose_dtype, stored_matrix_dtype
from .random_init import random_tensors, write_random_model, write_random_gguf

__all__ = ["OnDemand", "SafetensorsFile", "SafetensorsError", "write_safetensors", "GGUFFile", "GGUFError", "write_gguf",
           "ParamSpec", "WeightError", "read_checkpoint", "check_tensors", "place_tensor", "load_into", "choose_dtype", "stored_matrix_dtype",
           "random_tensors", "write_random_model", "write_random_gguf"]
