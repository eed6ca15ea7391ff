from .safetensors_io import SafetensorsStore, SafetensorsError, save_safetensors
from .loader import WeightError, load_tensors, load_state, check_against, target_dtype
from .random_init import write_random_model, random_state, random_tensor

__all__ = ["SafetensorsStore", "SafetensorsError", "save_safetensors", "WeightError", "load_tensors",
           "load_state", "check_against", "target_dtype", "write_random_model", "random_state", "random_tensor"]
