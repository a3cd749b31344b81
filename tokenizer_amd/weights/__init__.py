from .loader import UnexpectedTensors, WeightError, load_weights, stored_form, weight_path
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, save_safetensors

__all__ = ["UnexpectedTensors", "WeightError", "load_weights", "stored_form", "weight_path", "random_tensor", "random_tensors",
           "write_random_model", "SafetensorsError", "SafetensorsFile", "save_safetensors"]
