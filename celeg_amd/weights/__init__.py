from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .loader import Checkpoint, WeightError, check_tensors, load_tensors
from .random_init import write_random_model, random_tensors, random_tensor

__all__ = ["SafetensorsFile", "SafetensorsError", "write_safetensors", "Checkpoint",
           "WeightError", "check_tensors", "load_tensors", "write_random_model",
           "random_tensors", "random_tensor"]
