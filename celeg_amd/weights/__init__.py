from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .random_init import write_random_model, random_tensors, random_tensor
from .checks import WeightError, check_folder

__all__ = ["SafetensorsFile", "SafetensorsError", "write_safetensors", "write_random_model",
           "random_tensors", "random_tensor", "WeightError", "check_folder"]
